// Host-side policy shared by the forward and the backward dispatch: tile sizes,
// launch geometry, where the tensors sit on the alignment grid, and when rows
// are split over workgroups or packed into groups.
#ifndef ASCAN_POLICY_H_
#define ASCAN_POLICY_H_

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <type_traits>

#include "ascan.h"
#include "dispatch.h"
#include "gate.h"
#include "split.h"
#include "traits.h"

namespace ascan {
namespace {

// Blocks (64 vectors = 1 KiB of a tensor each) per wave and tile step:
//   U / UB    forward / backward kernels of regular shapes: 4 KiB of each
//             tensor per wave, except the complex backward kernel (its three
//             inputs plus complex temporaries would spill);
//   UG / UBG  the same for the kernels that carry masking code (rows of
//             arbitrary start and length), which need registers for the masks.
template <class Tr> struct Tuning;
template <> struct Tuning<TraitsF32> { static constexpr int U = 4, UG = 4, UB = 4, UBG = 2; };
template <> struct Tuning<TraitsBF16> { static constexpr int U = 4, UG = 2, UB = 4, UBG = 2; };
template <> struct Tuning<TraitsF16> { static constexpr int U = 4, UG = 2, UB = 4, UBG = 2; };
template <> struct Tuning<TraitsC64> { static constexpr int U = 4, UG = 4, UB = 2, UBG = 2; };
template <> struct Tuning<TraitsC64RealTokens> : Tuning<TraitsC64> {};

// The same four for split rows (forward regular / general, backward regular /
// general).  A swept tile has a fixed cost (ticket, look-back, barriers), so the real
// dtypes take 4 KiB per wave in every swept kernel, the ones with masking code included
// (which fit their registers: wave 0 parks its vectors in LDS during the look-back, and a
// sub-tile that holds nothing of the row is skipped); the complex kernels keep 2 KiB, except
// the mask-free forward kernel, whose raw vectors all wait for pass 2 in LDS (forward_kernel.h;
// the backward kernel with its gate and gradient vectors there and 4 KiB per wave spills 48
// bytes and is no faster: (8,768,65536) 2.74 -> 2.71 ms, (8,768,32768) 1.31 -> 1.35,
// (4,1024,8192) 0.228 -> 0.241).
// (8 KiB per wave in the fp32 forward kernel, half as many tiles: 6.35-6.41 TB/s at
// (8,1536,65536) against 6.5-6.56, and 40 bytes of scratch.)
template <class Tr> struct SplitTuning {
    static constexpr int U = Tuning<Tr>::U, UG = Tuning<Tr>::UG, UB = Tuning<Tr>::UB, UBG = Tuning<Tr>::UBG;
};
template <> struct SplitTuning<TraitsF32> { static constexpr int U = 4, UG = 4, UB = 4, UBG = 4; };
template <> struct SplitTuning<TraitsBF16> { static constexpr int U = 4, UG = 4, UB = 4, UBG = 4; };
template <> struct SplitTuning<TraitsF16> { static constexpr int U = 4, UG = 4, UB = 4, UBG = 4; };
template <> struct SplitTuning<TraitsC64> { static constexpr int U = 4, UG = 2, UB = 2, UBG = 2; };
template <> struct SplitTuning<TraitsC64RealTokens> : SplitTuning<TraitsC64> {};

// Launch geometry: W waves per row, R rows per workgroup (W*R <= 16).
struct Plan {
    int waves_per_row;
    int rows_per_block;
};

int env_int(const char* name) {
    const char* s = getenv(name);
    return s ? atoi(s) : 0;
}

// Optional overrides for tuning runs, read once per process:
// ASCAN_WAVES_PER_ROW in {1,2,4,8,16}, ASCAN_ROWS_PER_BLOCK in {1,2,4,8,16}.
const Plan& forced_plan() {
    static const Plan p = [] {
        auto pow2 = [](int n) { return (n == 1 || n == 2 || n == 4 || n == 8 || n == 16) ? n : 0; };
        return Plan{pow2(env_int("ASCAN_WAVES_PER_ROW")), pow2(env_int("ASCAN_ROWS_PER_BLOCK"))};
    }();
    return p;
}

// Measured on MI355X: what counts is how few rows are being streamed at any
// one time.  With every wave on its own row the memory system sees thousands
// of concurrent streams and tops out near 5.0 TB/s; with 16 waves marching
// along one row it reaches 5.6-6.1 TB/s.  So a row
// gets as many waves as it has sub-tiles (up to 16).  Short rows keep small
// workgroups (256 threads, several rows each): packing more short rows into
// one large workgroup measured slower.
//
// `trim`: a row is scanned in whole tiles of w sub-tiles, and the last tile may be mostly empty
// (20000 bf16 elements in tiles of 16384: the second tile is a fifth full).  Waves without
// any of the row in their sub-tile only pass the carry on, so the empty part costs little
// arithmetic, but every tile step costs a round trip to memory and a barrier, and with 16 waves
// per row nothing else runs on the compute unit meanwhile.  Measured over T = 2500..45000 with
// every plan forced in turn (16-bit at (8,1536,T), complex64 at (8,768,T)), the fastest plan is
// the widest one that (a) leaves at most a third of its wave slots empty (a quarter with 16 waves), (b) is not a single tile
// step with more than a fifth of it empty (two steps of half the width do better: the second
// step's loads overlap the first one's stores), and (c) is not a single step of 16 waves at all.
// That rule is within 4 % of the best plan at every length tried but one (bf16 T = 6000, 12 %).
// The fp32 kernels do less arithmetic per byte and are within 2 % of their best plan untrimmed
// (fp32 T = 9000 forward: 6 %), so they keep w -- except the interpolating gate's backward kernel.
template <class Tr>
constexpr bool kTrimPlan = Tr::kNarrow || !std::is_same<typename Tr::V, float>::value;

Plan choose_plan(int64_t T, int64_t sub, int64_t element_bytes, bool trim) {
    const Plan& forced = forced_plan();
    // one wave per 4 KiB of row, but never more waves than sub-tiles
    int w = 1;
    while (w < kMaxWavesPerBlock && (int64_t)w * 4096 < T * element_bytes && (int64_t)w * sub < T) w *= 2;
    if (trim) {
        auto steps = [&](int waves) { return (T + (int64_t)waves * sub - 1) / ((int64_t)waves * sub); };
        // wave slots (of `sub` elements each) a row occupies over all its tile steps
        auto slots = [&](int waves) { return steps(waves) * waves; };
        auto acceptable = [&](int waves) {
            const int64_t covered = slots(waves) * sub;
            if (waves == kMaxWavesPerBlock ? covered * 3 > T * 4 : covered * 2 > T * 3) return false;  // (a)
            if (steps(waves) == 1 && waves > 1 && covered * 5 > T * 6) return false;        // (b)
            if (steps(waves) == 1 && waves == kMaxWavesPerBlock && covered > T) return false;  // (c)
            return true;
        };
        int best = w;
        bool found = false;
        for (int v = w; v >= 1 && !found; v /= 2) {
            if (acceptable(v)) {
                best = v;
                found = true;
            } else if (slots(v) < slots(best)) {
                best = v;  // nothing acceptable so far: remember the plan with the fewest slots
            }
        }
        w = best;
    }
    if (forced.waves_per_row) w = forced.waves_per_row;
    int r = w >= 4 ? 1 : 4 / w;
    if (forced.rows_per_block) r = forced.rows_per_block;
    if (w * r > kMaxWavesPerBlock) r = kMaxWavesPerBlock / w;
    return Plan{w, r};
}

// Offset of an address from the grid boundary below it, in elements of
// `elem_bytes` bytes; boundaries are `grid` elements apart.  Tensors whose first
// elements have the same lead line up vector by vector, row by row.
int lead_of(const void* p, size_t elem_bytes, int grid) {
    return (int)((reinterpret_cast<uintptr_t>(p) / elem_bytes) % (unsigned)grid);
}

// The grid rows are addressed from (elements between boundaries) and where the
// call's tensors sit on it.
struct Lead {
    int grid;   // 128 bytes of states when all tensors agree there, else one 16-byte vector
    int lead;   // of the first tensor
    bool same;  // all tensors share `lead` on `grid`
};

template <class Tr, size_t N>
Lead find_lead(const void* const (&state_like)[N], const void* token_like) {
    constexpr size_t kElem = sizeof(typename Tr::S);
    for (int grid : {(int)(128 / kElem), Tr::EPV}) {
        const int lead = lead_of(state_like[0], kElem, grid);
        bool same = lead_of(token_like, sizeof(typename Tr::TokS), grid) == lead;
        for (size_t i = 1; i < N; ++i) same = same && lead_of(state_like[i], kElem, grid) == lead;
        if (same || grid == Tr::EPV) return Lead{grid, lead, same};
    }
    return Lead{Tr::EPV, 0, false};  // not reached
}

// Launches through hipLaunchKernel so that the launch's own status comes back
// (the <<<>>> form reports through the thread's sticky last-error slot, which
// may hold an error of the caller's).
template <class... Args>
hipError_t launch(void (*kernel)(Args...), unsigned blocks, unsigned threads, hipStream_t stream, Args... args) {
    void* argv[] = {static_cast<void*>(&args)...};
    return hipLaunchKernel(reinterpret_cast<const void*>(kernel), dim3(blocks), dim3(threads), argv, 0, stream);
}

inline int launch_status(hipError_t e) {
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ASCAN_ERR_LAUNCH;
    }
    return ASCAN_OK;
}


// Split-row policy.  With a table from the caller, the tiles of all rows can be
// swept in memory order by persistent 16-wave workgroups (split.h).  That is the only
// way to occupy the GPU when there are fewer rows than compute units, and for long
// rows it is faster than one workgroup walking each row whatever their number --
// where the tiles are large and not mostly empty.  Measured at (8,1536,T), forward +
// backward, % of the 8 TB/s peak, row walk -> sweep: fp32 T = 16384 72 -> 81,
// 32768 72 -> 82, 49152 65 -> 82, 65536 73 -> 82.5, and with rows of any start and
// length 65533 68 -> 81, 100000 -> 82, 50001 -> 82, 33000 / 36000 70 -> 80, 20000 /
// 22000 74 -> 78, 17000 (tiles 52 % full) 74 -> 75; a row of half a tile (8192)
// 75 -> 72 in a tile of its own, though its backward pass alone gains (want_split),
// and 77 -> 80 with two rows to a tile (sweep_rows_per_tile).
// bf16 T = 32768 72 -> 81, 65536 74 -> 82, 49152 73 -> 78, 100000 / 131071 69 -> 74 /
// 75, 45000 (tiles 69 % full) 71 -> 72, but 40000 (61 %) 72 -> 70 and 35000 (53 %)
// 70 -> 61.  complex64 (8,768,65536) 71 -> 70 with both kernels swept (64 KiB forward
// tiles, which spill; 64 with 32 KiB ones), 73 with the backward kernel alone
// (complex_rows_swept).  A tile costs a ticket, a look at the table and three
// barriers, about 2.4 us in which its compute unit requests nothing, whatever its
// size: all swept kernels of the real dtypes take 64 KiB tiles (4 KiB per wave).
// ASCAN_SPLIT_MAX_ROWS (0 = never split) and ASCAN_SPLIT_MIN_ROW_BYTES (split every
// row at least that long) override the rule, read once.
constexpr int kSplitWaves = 16;
constexpr int64_t kSweepTileBytes = 64 * 1024;  // of one tensor, 16 waves x 4 KiB

int64_t env_int64(const char* name, int64_t fallback) {
    const char* s = getenv(name);
    return s ? (int64_t)atoll(s) : fallback;
}
int64_t split_max_rows() {
    static const int64_t v = env_int64("ASCAN_SPLIT_MAX_ROWS", INT64_MAX);
    return v;
}
int64_t split_forced_min_row_bytes() {
    static const int64_t v = env_int64("ASCAN_SPLIT_MIN_ROW_BYTES", 0);
    return v;
}

// Longest single wait of a workgroup for an earlier tile, in 100 MHz ticks
// (default 2 s; ASCAN_SPLIT_WAIT_US overrides, read once).
unsigned long long split_wait_limit() {
    static const unsigned long long v = [] {
        const char* s = getenv("ASCAN_SPLIT_WAIT_US");
        const unsigned long long us = s ? strtoull(s, nullptr, 10) : 2000000ull;
        return us * 100ull;
    }();
    return v;
}

enum class SweepClass { kF32, kNarrow, kComplex };

// ASCAN_SWEEP_ROWS (sweep_rows_per_tile below), read once; -1 when unset.
int sweep_rows_mode() {
    static const int v = getenv("ASCAN_SWEEP_ROWS") ? env_int("ASCAN_SWEEP_ROWS") : -1;
    return v;
}
constexpr int64_t kSweepRowsMinBytes = 256ll << 20;  // of one tensor
constexpr int64_t kShortRowsSweptMinBytes = 128ll << 20;  // of one tensor (want_split)
template <class Tr>
constexpr SweepClass kSweepClass = Tr::kNarrow ? SweepClass::kNarrow
                                               : (std::is_same<typename Tr::V, float>::value ? SweepClass::kF32
                                                                                             : SweepClass::kComplex);

// complex64: many rows.  The forward kernel with masking code loses when swept whatever the shape (32 KiB
// tiles, twice the arithmetic per byte: (8,768,65536) 1.65 -> 2.05 ms); the mask-free one, with 64 KiB tiles
// and its raw vectors in LDS between the passes, gains on rows of two tiles and more ((8,768,T),
// T = 65536 / 32768 / 16384: 1.64 -> 1.59, 0.81 -> 0.78, 0.405 -> 0.400; one tile, (4,1024,8192),
// 0.150 -> 0.154).  The mask-free backward kernel, which requests the states behind pass 1, gains on rows
// of one tile and more when there are more than two per compute unit: (8,768,65536) 2.89 -> 2.73 ms,
// (8,768,32768) 1.41 -> 1.31, (4,1024,8192) 0.235 -> 0.219, (1,2048,32768) 0.476 -> 0.444, (1,512,32768)
// 0.129 -> 0.123; 256 rows lose (0.124 -> 0.130) and so does the kernel with masking code ((8,768,65533)
// 2.94 -> 3.18).  Rows of 1 MiB and more were level when every lane walked the tile's wave totals and the
// forward kernel took all rows in memory order; now they gain too, forward + backward, % of peak:
// (2,1536,131072) 71.1 -> 73.3, (1,1536,262144) 68.7 -> 72.3, (1,768,524288) 67.3 -> 72.4, (1,600,1048576)
// 62 -> 73, (1,512,131072) 70.5 -> 71.8, (1,1024,131072) 71.2 -> 73.0.
bool complex_rows_swept(int64_t rows, int64_t row_bytes) { return rows >= 512 && row_bytes >= kSweepTileBytes; }

// Too few rows to occupy the compute units with one workgroup each: with up to 64
// rows two tiles per row already pay; up to 128, four.
bool too_few_rows(int64_t rows, int64_t ntiles) {
    return (ntiles >= 2 && rows <= 64) || (ntiles >= 4 && rows <= 128);
}

// `row_bytes`: one row of states; `tile_bytes`, `ntiles`: of the kernel that would run;
// `act`: its gate; `forward`: the forward kernel (3 tensors per tile) or the backward one
// (5 or 6); `mask_free`: the kernel for rows of whole tiles on the grid.  A compute unit
// holds one swept workgroup, so what a tile costs in arithmetic is not hidden behind another
// workgroup's loads: the 16-bit forward kernels that form a token from the gate, a second
// activation for eight elements per vector, lose when swept (bf16 (8,1536,65536), ms, whole
// rows -> swept: interpolating gate 0.80 -> 0.86, normalised exponential 0.81 -> 0.94), and so
// does a sigmoid evaluated in both passes (0.79 -> 0.92), as the copies with masking code
// do; the mask-free kernel keeps the gates of pass 1 in LDS and gains (0.79 -> 0.75, fp16
// 0.79 -> 0.73; T = 32768 0.40 -> 0.39 / 0.37), like the plain exponential and the fp32
// kernels of all gates (72 -> 78-82 % of peak).  A forward kernel with 32 KiB tiles loses
// (the normalised exponential gate's with masking code, fp32: 6.0 -> 5.3 TB/s).  The backward kernels
// move five or six tensors per tile, do well with 32 KiB of each, request the states behind
// pass 1 so that they travel while the tile looks at the table, and keep the activated gates
// of pass 1 in LDS (backward_kernel.h).  Swept, the mask-free 16-bit ones gain (bf16
// (8,1536,65536) backward, ms, whole rows -> swept: sigmoid 1.46 -> 1.24, interpolating gate
// 1.73 -> 1.45, normalised exponential 1.72 -> 1.49; T = 32768 0.79 -> 0.63, 0.93 -> 0.74,
// 0.90 -> 0.75; fp16 alike).  With masking code (T = 65533) the sigmoid's gains, 1.49 -> 1.39,
// the two with values do not: interpolating gate 1.82 -> 1.85, normalised exponential
// 1.79 -> 1.82.
bool want_split(SweepClass c, int64_t rows, int64_t row_bytes, int64_t tile_bytes, int64_t ntiles, int act, bool forward,
                bool mask_free) {
    if (rows > split_max_rows()) return false;
    if (too_few_rows(rows, ntiles)) return true;
    if (split_forced_min_row_bytes() > 0) return row_bytes >= split_forced_min_row_bytes();
    if (forward && tile_bytes < kSweepTileBytes) return false;
    // 32 KiB tiles (the backward kernels of the gates with values) on rows shorter than 64 KiB: one workgroup
    // per row does badly there (fp32 interpolating gate, (8,1536,T) backward, ms, whole rows -> swept:
    // T = 8192 0.41 -> 0.37, 10000 0.52 -> 0.50, 12288 0.62 -> 0.58, 14000 0.74 -> 0.64; (16,1536,8192)
    // 0.88 -> 0.74; bf16 (8,1536,16384) 0.41 -> 0.37), but a sweep needs a launch worth its start:
    // (4,1536,8192) 0.203 -> 0.192, (2,1536,8192) 0.102 -> 0.103, (1,1536,8192) 0.052 -> 0.058.
    if (tile_bytes < kSweepTileBytes && row_bytes < kSweepTileBytes &&
        (row_bytes < tile_bytes || rows * row_bytes < kShortRowsSweptMinBytes)) {
        return false;
    }
    // How full the row's tiles are.  The remainder tile costs little (it is the first of its row in scan
    // order and its empty sub-tiles are skipped) but not nothing, and a row shorter than a tile leaves
    // part of its only tile's workgroup idle.  Measured, fp32 (8,1536,T), TB/s whole rows -> swept:
    // forward T = 8192 6.1 -> 5.0, 10000 5.86 -> 5.77, 12000 6.08 -> 6.24, 13000 6.08 -> 6.26, 14000 6.1 -> 6.2,
    // 17000 6.0 -> 5.9, 20000 5.9 -> 6.2;
    // backward (320 KiB per full tile rather than 192) 8192 6.0 -> 6.2, 10000 6.1 -> 6.3, 12000 6.0 -> 6.4,
    // 17000 5.9 -> 6.3; bf16 35000 (53 %) 70 -> 61 % of peak, 40000 (61 %) 72 -> 70, 45000 (69 %) 71 -> 72,
    // 24000 and 16384 (one tile, 73 and 50 % full) 71 -> 69 and 78 -> 63.
    const int64_t percent_full = row_bytes * 100 / (ntiles * tile_bytes);
    switch (c) {
        case SweepClass::kF32: return percent_full >= (forward ? (ntiles == 1 ? 73 : 55) : 50);
        case SweepClass::kNarrow:
            return row_bytes >= tile_bytes && percent_full >= 66 &&
                   (act == kGateIdentity || act == kGateExp || (act == kGateSigmoid && (mask_free || !forward)) ||
                    (gate_takes_values(act) && mask_free && !forward));
        default:
            return mask_free && complex_rows_swept(rows, row_bytes) && (!forward || row_bytes >= 2 * kSweepTileBytes);
    }
}

// Whether some kernel of a call of this shape may want the table with its records (`ntiles_most`:
// with the smallest tile any kernel uses): what ascan_workspace_bytes goes by.  `forward_only`: the
// identity gate's forward kernel alone (the entry point with the table in the library's own array).
bool may_split(SweepClass c, int64_t rows, int64_t row_bytes, int64_t ntiles_most, bool forward_only) {
    if (rows > split_max_rows()) return false;
    if (too_few_rows(rows, ntiles_most)) return true;
    if (split_forced_min_row_bytes() > 0) return row_bytes >= split_forced_min_row_bytes();
    const bool half_tile_rows = row_bytes == kSweepTileBytes / 2 && rows * row_bytes >= kSweepRowsMinBytes;
    switch (c) {
        case SweepClass::kF32:  // a backward kernel takes half-full tiles, a forward kernel does not
            return forward_only ? row_bytes > kSweepTileBytes / 2 : row_bytes >= kSweepTileBytes / 2;
        case SweepClass::kNarrow: return row_bytes >= kSweepTileBytes || (!forward_only && half_tile_rows);
        default: return !forward_only && complex_rows_swept(rows, row_bytes);
    }
}
// Rows swept two to a tile by the forward kernel need the ticket, not the records.
bool forward_needs_ticket_only(SweepClass c, int64_t rows, int64_t row_bytes) {
    return c != SweepClass::kComplex && rows <= split_max_rows() && sweep_rows_mode() != 0 &&
           row_bytes == kSweepTileBytes / 2 && rows * row_bytes >= kSweepRowsMinBytes;
}

// Rows of exactly half a swept tile, starting on the grid: two whole rows per tile of a
// kSweepRows launch, each on eight waves (returns the rows per tile, or 0).  `sub`: the
// elements per wave of the mask-free kernel that would run.  The tiles are full and no
// tile waits for another, so the sweep runs as for rows of one full tile -- but a launch
// costs the table's reset and the filling of 256 persistent workgroups, which shorter
// rows (several per tile work just as well) and small tensors do not earn back.
// Measured, forward + backward, % of peak, whole rows -> swept: fp32 (B,1536,8192) B = 16
// 77.7 -> 81.6, 8 77.2 -> 79.8, 4 76.8 -> 77.0, 2 73.8 -> 71.6; (8,1536,4096) 79.8 -> 76.7,
// (8,1536,2048) 78.3 -> 71.6; bf16 (8,1536,16384) 77.2 -> 79.1, (4,1536,16384) 77.9 -> 75.5;
// fp16 (8,1536,16384) 76.4 -> 79.9.  With a gate, ms forward + backward at those shapes:
// fp32 sigmoid 0.541 -> 0.510, exp 0.535 -> 0.509, bf16 sigmoid 0.525 -> 0.627, exp
// 0.514 -> 0.558 (a compute unit holds one swept workgroup and does not hide the 16-bit
// kernels' gate arithmetic behind another's loads).  Rows that leave sub-tiles partly
// empty lose (fp32 T = 6000 77.3 -> 75.2, bf16 12000 73.9 -> 63.3), and so do tiles handed
// out by workgroup index instead of by ticket (70 %) and tickets drawn a tile ahead, behind
// the loads (77.5 % at T = 8192: no tile waits for another here, but the stretch of memory
// in flight is twice as long).
// ASCAN_SWEEP_ROWS = 0 / 1 (never / whenever rows divide a tile) overrides the rule.
int sweep_rows_per_tile(SweepClass c, int64_t rows, int64_t T, int64_t elem_bytes, int64_t sub, int act) {
    if (c == SweepClass::kComplex || T % sub != 0 || rows > split_max_rows() || sweep_rows_mode() == 0) return 0;
    const int64_t row_waves = T / sub;
    if (row_waves * 2 > kSplitWaves || kSplitWaves % row_waves != 0) return 0;
    const int per_tile = (int)(kSplitWaves / row_waves);
    if (sweep_rows_mode() == 1) return per_tile;
    if (per_tile != 2 || rows * T * elem_bytes < kSweepRowsMinBytes) return 0;
    if (c != SweepClass::kF32 && act != kGateIdentity) return 0;
    return per_tile;
}

size_t split_bytes(int64_t rows, int64_t ntiles) {
    return sizeof(SplitHeader) + sizeof(SplitTicket) + (size_t)rows * (size_t)ntiles * sizeof(SplitRecord);
}

// The table is usable for this launch: aligned, large enough, and the tickets fit the
// 32 bits the kernels turn into (row, tile).
bool workspace_fits(const Workspace& ws, int64_t rows, int64_t ntiles) {
    return ws.ptr != nullptr && (reinterpret_cast<uintptr_t>(ws.ptr) % alignof(SplitRecord)) == 0 &&
           rows <= 2147483647LL / ntiles && ws.bytes >= split_bytes(rows, ntiles);
}

hipError_t reset_split_table(const Workspace& ws, int64_t rows, int64_t ntiles, hipStream_t stream) {
    const size_t nwords = split_bytes(rows, ntiles) / sizeof(uint32_t);
    const unsigned blocks = (unsigned)((nwords + 255) / 256);
    return launch(split_reset_kernel, blocks, 256u, stream, static_cast<uint32_t*>(ws.ptr), nwords,
                  split_wait_limit());
}

// Number of workgroups of `kernel` (of `threads` threads, no dynamic LDS) the
// current device holds at one time, `most_per_cu` per compute unit at most (the same
// at every call for one kernel).  Queried once per kernel and device.
// The swept kernels that hold several rows per tile need no registers for a look-back
// and would fit twice, but run one workgroup per compute unit like the others: measured,
// fp32 (8,1536,8192) forward 6.3 TB/s with one, 5.9 with two.
template <class K>
unsigned resident_workgroups(K kernel, int threads, int most_per_cu) {
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return 0;
    constexpr int kMaxDevices = 64;
    static std::atomic<unsigned> cache[kMaxDevices];  // 0 = not queried yet; one array per kernel instantiation
    if (device < 0 || device >= kMaxDevices) return 0;
    unsigned known = cache[device].load(std::memory_order_relaxed);
    if (known == 0) {
        int per_cu = 0, cus = 0;
        if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, kernel, threads, 0) != hipSuccess ||
            hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess ||
            per_cu <= 0 || cus <= 0) {
            return 0;
        }
        if (per_cu > most_per_cu) per_cu = most_per_cu;
        known = (unsigned)per_cu * (unsigned)cus;
        cache[device].store(known, std::memory_order_relaxed);
    }
    return known;
}

// Tiles per row as the kernels count them (tiles_per_row on the device), and the
// distance from the grid boundary they address rows from to a row's first element, at most.
inline int host_head(int64_t T, bool regular, const Lead& at) {
    return regular ? 0 : (T % at.grid == 0 ? at.lead : at.grid - 1);
}
template <class Tr>
int64_t host_tiles_per_row(int64_t T, int64_t tile, bool regular, const Lead& at) {
    return (T + host_head(T, regular, at) + tile - 1) / tile;
}

// Packed-row policy.  Rows shorter than kPackedMaxRowBytes (of states) are
// scanned in groups, one group per 4-wave workgroup; a group fills one tile of
// the general kernel, counting the lead of its first element, and when possible
// is a whole number of 128-byte lines long so that every group starts on the
// grid like the first.  ASCAN_PACKED_MAX_ROW_BYTES overrides the limit (0
// switches packing off), read once.
constexpr int kPackedWaves = 4;
// The 16-bit backward kernels do better with 8-wave workgroups once rows reach
// 512 bytes (measured, 4 -> 8 waves: bf16 (64,4096,256) 5.1 -> 5.6 TB/s,
// (16,4096,1000) 5.4 -> 5.7, (64,4096,500) 5.5 -> 5.8; shorter rows and the
// forward kernels lose 5-15 %, fp32 and complex64 gain or lose a few per cent
// depending on the row length).
constexpr int kPackedWavesWide = 8;
constexpr int64_t kPackedWideRowBytes = 512;
constexpr int64_t kPackedWideMinGroups = 2048;  // fewer, larger workgroups only when there are plenty (8 per compute unit)
constexpr int64_t kPackedMaxRowBytesDefault = 2048;

int64_t packed_max_row_bytes() {
    static const int64_t v = [] {
        const char* s = getenv("ASCAN_PACKED_MAX_ROW_BYTES");
        return s ? (int64_t)atoll(s) : kPackedMaxRowBytesDefault;
    }();
    return v;
}

int64_t gcd64(int64_t a, int64_t b) {
    while (b != 0) {
        const int64_t t = a % b;
        a = b;
        b = t;
    }
    return a;
}

// Rows per group for rows of T elements, tiles of `tile` elements and a grid of
// `grid` elements; 0 when rows of this length are not packed.
int packed_group(int64_t rows, int64_t T, int64_t element_bytes, int64_t tile, int grid) {
    if (rows < 2 || T * element_bytes >= packed_max_row_bytes()) return 0;
    int64_t group = (tile - grid) / T;
    if (group < 2) return 0;
    // a whole number of grid cells per group, so that every group starts on the grid like
    // the first, unless that would leave more than 15 % of the tile empty
    const int64_t whole_lines = grid / gcd64(T, grid);  // rows per whole number of grid cells
    const int64_t whole = group - group % whole_lines;
    if (whole > 0 && whole * 100 >= group * 85) group = whole;
    return (int)group;
}

// Memory-access flavour of a launch.
//   kRegular    : every row starts on a grid boundary and is a whole number
//                 of tiles long, so every sub-tile is full: the kernel carries
//                 no masking code at all (the common case: T a power of two).
//   kVector     : all tensors share one offset from the grid; rows may start
//                 anywhere and have any length.  Whole-vector accesses except
//                 where a vector straddles a row end.
//   kElementwise: tensors at different offsets inside a 16-byte vector.
enum class Access { kRegular, kVector, kElementwise };

Access choose_access(bool same_lead, int lead, int64_t T, int64_t tile) {
    if (!same_lead) return Access::kElementwise;
    if (lead == 0 && T % tile == 0) return Access::kRegular;
    return Access::kVector;
}

// Kernels with a gate non-linearity exist for the real dtypes, forward in time.
template <class Tr>
constexpr bool kHasSigmoid = std::is_same<typename Tr::V, float>::value;

// Calls f(std::integral_constant<int, ACT>) for the gate code `act`, which the
// entry points have validated against the dtype.  SCAN_FORWARD = false (reverse
// scans and their backward pass) has the identity gate only.
template <class Tr, bool SCAN_FORWARD = true, class F>
hipError_t with_gate(int act, F&& f) {
    if constexpr (kHasSigmoid<Tr> && SCAN_FORWARD) {
        if (act == kGateSigmoid) return f(std::integral_constant<int, kGateSigmoid>{});
        if (act == kGateSigmoidLerp) return f(std::integral_constant<int, kGateSigmoidLerp>{});
        if (act == kGateExp) return f(std::integral_constant<int, kGateExp>{});
        if (act == kGateExpNorm) return f(std::integral_constant<int, kGateExpNorm>{});
    }
    return f(std::integral_constant<int, kGateIdentity>{});
}

// The backward kernel of a gate with values holds a fourth input tensor in
// registers and takes 2 KiB per wave and tile at most.
template <int ACT>
constexpr int backward_blocks(int blocks) {
    return kGateTakesValues<ACT> && blocks > 2 ? 2 : blocks;
}
inline int backward_blocks_of(int act, int blocks) { return gate_takes_values(act) && blocks > 2 ? 2 : blocks; }

// The split-row forward kernel of the normalised exponential gate (two activations
// per element next to the look-back's registers) takes 2 KiB per wave and tile as well --
// except the mask-free fp32 one, which keeps gate and token of pass 1 in LDS and needs
// no registers for a second evaluation (79 against 113).
template <class Tr, int ACT, bool REGULAR>
constexpr int forward_split_blocks(int blocks) {
    constexpr bool kept_in_lds = REGULAR && std::is_same<typename Tr::S, float>::value;
    return ACT == kGateExpNorm && !kept_in_lds && blocks > 2 ? 2 : blocks;
}
template <class Tr>
inline int forward_split_blocks_of(int act, int blocks, bool regular) {
    const bool kept_in_lds = regular && std::is_same<typename Tr::S, float>::value;
    return act == kGateExpNorm && !kept_in_lds && blocks > 2 ? 2 : blocks;
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_POLICY_H_
