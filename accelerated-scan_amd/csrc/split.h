// Rows split over many workgroups: the table in global memory, the hand-out
// of tiles by ticket and the decoupled look-back.

#ifndef ASCAN_SPLIT_H_
#define ASCAN_SPLIT_H_

#include "carry.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Split rows: the tiles of all rows are handed out in memory order, one tile to
// one workgroup at a time, and the state entering a tile comes from the
// workgroups of the row's earlier tiles through a small table in global memory.
//
// Order.  There is one ticket counter for the whole launch: ticket n is tile
// n % ntiles of row n / ntiles, so the resident workgroups together sweep the
// tensors front to back, each taking the next 16-wave tile whenever it is done
// with its last.  Measured on MI355X with kernels that only move the bytes
// (3 reads + 2 writes, 3.2 GB per tensor): one workgroup walking each 256 KiB
// row 5.56 TB/s (5.1 with rows 192 KiB apart); this sweep, with a wait on the
// row's earlier tiles before a tile's stores, 6.46 TB/s (6.25).  What the sweep
// buys is the compact stretch of memory in flight at any one time; what it
// costs is one look at the table per tile, whose latency (about 3 us under
// load, same XCD or not) is idle time of one compute unit that the others fill.
// A ticket is drawn when the workgroup is ready for the tile, never ahead: a
// tile held back by its owner's previous tile stalls every later tile of the row.
//
// Long rows.  In memory order the tiles in flight at one time -- one per compute
// unit -- are a few whole rows when rows are long, so a tile has up to 63 earlier
// tiles of its window in flight beside it and waits for the slowest of them.  The
// forward kernel therefore hands out rows of 16 tiles and more in bands (band_rows
// below): ticket n of a band of R rows is tile n / R of the band's row n % R, so the
// tiles in flight are 256 / R consecutive tiles of each of R rows, and a tile waits
// for a handful.  A tile's earlier tiles still hold smaller tickets.  Measured, fp32
// forward, 3.2 GB per tensor, ms, memory order -> bands: 16 tiles per row 1.567 ->
// 1.53 (R = 64; 1.59-1.84 with R = 32), 32 tiles 1.62 -> 1.51 (R = 32; 1.52 with
// 64), 64 tiles 1.68 -> 1.54 (1.58 with 64, 1.60 with 128), 128 tiles 1.576 -> 1.52,
// bf16 64 tiles 1.73 -> 1.55.  The backward kernel, with five tensors per tile,
// prefers memory order: R = 32 / 64, 16 tiles 2.49 -> 2.9 / 2.61, 64 tiles 2.65 ->
// 2.62 / 2.72, 128 tiles 2.57 -> 2.63 / 2.69.
//
// Because tickets are taken in order, a tile is only ever waited for by
// workgroups that started after its owner did: progress never depends on a
// workgroup that has not been dispatched yet, whatever else is running on the
// GPU, and the launch size (what an idle GPU holds at once) is a matter of
// speed only.  Each wait is nevertheless bounded by a limit set by the host; a
// wait that runs out poisons the result with NaN and is counted in the header.
// Waiting time is summed from clock differences capped at 10 us each, so a
// stretch during which the whole kernel was not running does not count.
//
// Look-back.  The tiles of a row form windows of 64.  A workgroup publishes its
// tile's aggregate (A, X) as soon as it has it; the state entering tile k is the
// state entering k's window folded with the aggregates of the window's tiles
// before k -- lane i of wave 0 reads tile i of the window, all at once, and the
// 64 pairs are folded by the wave scan, in one fixed order.  The state entering
// a window is the inclusive state its predecessor's last tile publishes (the
// row's start for window 0), so the chain of waits is one hop per 64 tiles, and
// what a tile receives does not depend on timing: results are reproducible
// run to run.
// ---------------------------------------------------------------------------
struct SplitHeader {
    unsigned long long reserved0;
    unsigned long long wait_limit;  // longest single wait, in s_memrealtime ticks (100 MHz)
    unsigned int timeouts;          // waits that ran out
    unsigned int reserved[11];
};
static_assert(sizeof(SplitHeader) == 64, "header is 64 bytes");

// The ticket counter of the launch, on a cache line of its own.
struct alignas(64) SplitTicket {
    unsigned long long next;  // next tile to hand out: tile next % ntiles of row next / ntiles
    unsigned long long pad[7];
};
static_assert(sizeof(SplitTicket) == 64, "ticket line is 64 bytes");

// How a kernel's workgroups come by their work (template argument SPLIT of the scan kernels).
constexpr int kWholeRows = 0;  // a workgroup owns its rows from start to end
constexpr int kSweep = 1;      // tiles of all rows by ticket, in memory order; a row's tiles hand their state on
constexpr int kSweepRows = 2;  // the same for rows of at most half a tile: a tile holds several whole rows

// Rows per band for rows of `ntiles` tiles in the forward kernel; 0 = memory order.
__device__ __forceinline__ int band_rows(int64_t ntiles) { return ntiles >= 32 ? 32 : (ntiles >= 16 ? 64 : 0); }

constexpr unsigned long long kWaitStepCap = 1000;  // 10 us in 100 MHz ticks
constexpr int kSplitWindow = 64;                   // tiles per look-back window: one per lane

// One record per (row, tile).  Every field is a 64-bit word holding an fp32
// payload in its low half and a tag in its high half (0 = not written yet,
// 1 = valid), written and read with single relaxed device-scope atomics: the
// payload arrives together with its tag, so no fence (on this hardware a
// write-back or invalidate of a whole L2) is needed on either side.
struct alignas(64) SplitRecord {
    unsigned long long a[2];  // aggregate gate product of the tile (re, im)
    unsigned long long x[2];  // aggregate state of the tile from a zero start (re, im)
    unsigned long long p[2];  // inclusive state at the end of the tile (re, im); last tile of a window only
    unsigned long long pad[2];
};
static_assert(sizeof(SplitRecord) == 64, "record is 64 bytes");

constexpr unsigned long long kTagValid = 1ull << 32;

__device__ __forceinline__ void publish_word(unsigned long long* word, float v) {
    __hip_atomic_store(word, kTagValid | (unsigned long long)(unsigned int)f2i(v), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ unsigned long long peek_word(unsigned long long* word) {
    return __hip_atomic_load(word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool word_valid(unsigned long long w) { return (w >> 32) != 0ull; }
__device__ __forceinline__ float word_value(unsigned long long w) { return i2f((int)(unsigned int)w); }

__device__ __forceinline__ void publish(unsigned long long (&dst)[2], float v) { publish_word(&dst[0], v); }
__device__ __forceinline__ void publish(unsigned long long (&dst)[2], cfloat v) {
    publish_word(&dst[0], v.re);
    publish_word(&dst[1], v.im);
}
// Reads a field; returns false while any of its words is still unwritten.
__device__ __forceinline__ bool peek(unsigned long long (&src)[2], float& v) {
    const unsigned long long w = peek_word(&src[0]);
    v = word_value(w);
    return word_valid(w);
}
__device__ __forceinline__ bool peek(unsigned long long (&src)[2], cfloat& v) {
    const unsigned long long w0 = peek_word(&src[0]);
    const unsigned long long w1 = peek_word(&src[1]);
    v.re = word_value(w0);
    v.im = word_value(w1);
    return word_valid(w0) && word_valid(w1);
}
__device__ __forceinline__ float poison(float) { return __builtin_nanf(""); }
__device__ __forceinline__ cfloat poison(cfloat) { return cfloat{__builtin_nanf(""), __builtin_nanf("")}; }

// Clears the table before a split launch (a kernel rather than a memset so that
// the call can be captured into a graph).
__global__ void split_reset_kernel(uint32_t* words, size_t nwords, unsigned long long wait_limit) {
    const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    // the limit occupies words 2 and 3 of the header; every word has exactly one writer
    if (i < nwords) words[i] = i == 2 ? (uint32_t)wait_limit : (i == 3 ? (uint32_t)(wait_limit >> 32) : 0u);
}

// Layout of the table: header, the ticket line, one record per (row, tile).
__device__ __forceinline__ SplitTicket* split_ticket(SplitHeader* header) {
    return reinterpret_cast<SplitTicket*>(header + 1);
}
__device__ __forceinline__ SplitRecord* split_records(SplitHeader* header) {
    return reinterpret_cast<SplitRecord*>(split_ticket(header) + 1);
}

// Hands the workgroup its next tile, or returns false when none is left: thread 0
// draws the ticket, all threads of the workgroup call this together and get the
// same answer through `mailbox` (two words of LDS; the caller alternates between two mailboxes from
// call to call).  rows * ntiles is below 2^31.  `band`: rows per band, 0 for memory order.
//
// The ticket is drawn here, when the workgroup is ready to start on it, so tiles
// start in ticket order.  (Drawn a tile step ahead, behind the previous tile's
// loads, the fetch-add costs nothing, but then a tile starts whenever its owner's
// previous tile is done, and a workgroup held up in its look-back holds up the
// later tiles of the row it has the next ticket for: measured, a row's earlier
// tiles were ready 8-9 us after the later ones one time in ten, and the kernel lost
// a fifth of its speed.)  The draw, the mailbox and the barrier stay together in
// one straight piece of code, and what comes out of the mailbox is made wave-uniform
// explicitly, so that the loop around it branches uniformly: a thread-0-only draw
// at the far end of the loop body was compiled into a loop in which thread 0 left
// for its draw while the other lanes went on to read the mailbox it had yet to fill.
__device__ __forceinline__ bool take_split_tile(SplitHeader* header, int64_t rows, int64_t ntiles, int64_t& row,
                                                int64_t& k, int* mailbox, int band = 0) {
    if (threadIdx.x == 0) {
        const unsigned long long ticket = __hip_atomic_fetch_add(&split_ticket(header)->next, 1ull, __ATOMIC_RELAXED,
                                                                 __HIP_MEMORY_SCOPE_AGENT);
        int got_row = -1, got_k = -1;
        if (ticket < (unsigned long long)(rows * ntiles)) {
            const unsigned n = (unsigned)ticket, per_row = (unsigned)ntiles;
            if (band > 0) {
                const unsigned band_tiles = (unsigned)band * per_row;
                const unsigned b = n / band_tiles, i = n - b * band_tiles;
                const unsigned left = (unsigned)rows - b * (unsigned)band;  // the last band may hold fewer rows
                const unsigned in_band = left < (unsigned)band ? left : (unsigned)band;
                got_k = (int)(i / in_band);
                got_row = (int)(b * (unsigned)band + (i - (unsigned)got_k * in_band));
            } else {
                got_row = (int)(n / per_row);
                got_k = (int)(n - (unsigned)got_row * per_row);
            }
        }
        mailbox[0] = got_row;
        mailbox[1] = got_k;
    }
    __syncthreads();
    const int got_row = __builtin_amdgcn_readfirstlane(mailbox[0]);
    const int got_k = __builtin_amdgcn_readfirstlane(mailbox[1]);
    // (no second barrier: consecutive calls use alternate mailboxes, and a thread that is two calls
    // ahead has passed the barrier of the call in between, which every thread reaches after this read)
    if (got_row < 0) return false;
    row = got_row;
    k = got_k;
    return true;
}

// Waits (bounded) until both fields are published and returns them; false when the
// wait ran out.  The words of both fields are requested together: one round trip.
// The clock is only read once a look has found nothing.
template <class V>
__device__ __forceinline__ bool await_pair(unsigned long long (&fa)[2], unsigned long long (&fx)[2], V& a, V& x,
                                           unsigned long long limit) {
    unsigned long long waited = 0, last = 0;
    for (bool first = true;; first = false) {
        const bool has_a = peek(fa, a);
        const bool has_x = peek(fx, x);
        if (has_a && has_x) return true;
        const unsigned long long now = __builtin_amdgcn_s_memrealtime();
        if (!first) waited += now - last < kWaitStepCap ? now - last : kWaitStepCap;
        last = now;
        if (waited > limit) return false;
        __builtin_amdgcn_s_sleep(1);
    }
}
template <class V>
__device__ __forceinline__ bool await_field(unsigned long long (&field)[2], V& v, unsigned long long limit) {
    unsigned long long waited = 0, last = 0;
    for (bool first = true;; first = false) {
        if (peek(field, v)) return true;
        const unsigned long long now = __builtin_amdgcn_s_memrealtime();
        if (!first) waited += now - last < kWaitStepCap ? now - last : kWaitStepCap;
        last = now;
        if (waited > limit) return false;
        __builtin_amdgcn_s_sleep(1);
    }
}

// State entering scan-order tile k of a row, for wave 0 of the workgroup that
// owns the tile.  `mine` is the row's first record; (tileA, tileX) is this
// tile's aggregate and `row_start` the state entering tile 0.
template <class V>
__device__ __forceinline__ V split_look_back(SplitHeader* header, unsigned long long limit, SplitRecord* mine,
                                             int64_t k, int64_t ntiles, V tileA, V tileX, V row_start, int lane) {
    SplitRecord* rec = mine + k;
    const int64_t window = k & ~(int64_t)(kSplitWindow - 1);  // first tile of k's window
    const int r = (int)(k - window);                          // tiles of the window before k
    const bool closes_window = r == kSplitWindow - 1;
    const bool has_successor = k + 1 < ntiles;
    // the aggregate is read by the later tiles of the window, the inclusive state by the next window
    if (lane == 0 && has_successor && !closes_window) {
        publish(rec->a, tileA);
        publish(rec->x, tileX);
    }
    V carry_in = row_start;
    if (k > 0) {
        V A = vone<V>(), X = vzero<V>();
        bool late = false;
        if (lane < r) {
            SplitRecord* prev = mine + window + lane;
            late = !await_pair(prev->a, prev->x, A, X, limit);
        } else if (lane == kSplitWindow - 1 && window > 0) {
            // the state entering the window; lane 63 never holds an aggregate (r <= 63)
            late = !await_field((mine + window - 1)->p, X, limit);
        }
        if (__ballot(late)) {
            // a wait ran out: give up on this tile, visibly
            if (lane == 0) atomicAdd(&header->timeouts, 1u);
            carry_in = poison(carry_in);
        } else {
            const V entering = window > 0 ? read_lane<kSplitWindow - 1>(X) : row_start;
            if (lane == kSplitWindow - 1) X = vzero<V>();
            wave_scan_inclusive<false>(A, X);  // lanes past r hold the identity
            carry_in = vfma(read_lane<63>(A), entering, read_lane<63>(X));
        }
    }
    if (lane == 0 && has_successor && closes_window) publish(rec->p, vfma(tileA, carry_in, tileX));
    return carry_in;
}

// exchange_carries for a workgroup that owns a single tile of a split row: the
// tile carry comes from split_look_back instead of the previous loop iteration.
//
// Wave 0 looks back while it holds its sub-tile in registers like every other
// wave, and the look-back needs registers of its own.  `set_aside()` /
// `take_back()` are called by wave 0 only, around it: the kernels park their raw
// vectors in LDS there, which frees those registers without a trip through
// scratch memory.
// LANES: how the waves' totals are folded (below).
template <class V, int W, int U, bool LANES, class SetAside, class TakeBack>
__device__ __forceinline__ void exchange_carries_split(const V (&totA)[U], const V (&totX)[U], V& c, V* slots,
                                                       int w, int lane, SplitHeader* header, unsigned long long limit,
                                                       SplitRecord* mine, int64_t k, int64_t ntiles, V row_start,
                                                       SetAside set_aside, TakeBack take_back) {
    V TA = totA[0], TX = totX[0];
#pragma unroll
    for (int j = 1; j < U; ++j) {
        TX = vfma(TX, totA[j], totX[j]);
        TA = vmul(TA, totA[j]);
    }
    if (lane == 0) {
        slots[2 * w] = TA;
        slots[2 * w + 1] = TX;
    }
    __syncthreads();
    // aggregate of the waves before this one, and of the whole tile, from the identity
    V runA = vone<V>(), runX = vzero<V>();
    V mineA = runA, mineX = runX;
    if constexpr (LANES) {
        // lane i takes wave i's pair and four row-shift steps fold the W <= 16 of them, instead of every
        // lane walking through all W: a quarter of the instructions, one LDS read instead of W, and 30
        // registers fewer.  Measured at (8,1536,65536), ms, forward: fp32 1.50 -> 1.48, bf16 0.742 -> 0.732,
        // complex64 (8,768,65536) 1.61 -> 1.57, bf16 T = 131071 1.62 -> 1.57; the complex backward kernel
        // 2.74 -> 2.66; the backward kernels of the real dtypes lose, fp32 2.44 -> 2.46, bf16 1.235 -> 1.255,
        // bf16 T = 131071 2.68 -> 2.85, and walk as before.  (So do the kernels that own whole rows: with
        // fewer registers more of their workgroups share a compute unit, and more rows stream at a
        // time: fp32 (8,1536,65536) forward 1.62 -> 1.69 ms.)
        static_assert(W <= 16, "the waves of a tile fit one row of lanes");
        V A = vone<V>(), X = vzero<V>();
        if (lane < W) {
            A = slots[2 * lane];
            X = slots[2 * lane + 1];
        }
        scan_step<kRowShr1, 0xF, false>(A, X);
        scan_step<kRowShr2, 0xF, false>(A, X);
        scan_step<kRowShr4, 0xF, false>(A, X);
        scan_step<kRowShr8, 0xF, false>(A, X);
        runA = read_lane<W - 1>(A);
        runX = read_lane<W - 1>(X);
        const int wave = __builtin_amdgcn_readfirstlane(w);
        mineA = read_lane_at(shift_up1(A, vone<V>()), wave);
        mineX = read_lane_at(shift_up1(X, vzero<V>()), wave);
    } else {
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const V Ai = slots[2 * i];
            const V Xi = slots[2 * i + 1];
            mineA = vselect(i == w, runA, mineA);
            mineX = vselect(i == w, runX, mineX);
            runX = vfma(runX, Ai, Xi);
            runA = vmul(runA, Ai);
        }
    }
    V* carry_slot = slots + kSlotsPerBuffer;
    if (w == 0) {  // wave-uniform
        set_aside();
        const V carry_in = split_look_back(header, limit, mine, k, ntiles, runA, runX, row_start, lane);
        if (lane == 0) *carry_slot = carry_in;
        take_back();
    }
    __syncthreads();
    c = vfma(mineA, *carry_slot, mineX);
}

// The same for a swept tile that holds several whole rows (kSweepRows): the waves
// [first, first + waves of a row) scan one row, so a wave's prefix runs over the
// waves of its own row only and starts from that row's own state.  No tile depends
// on another, so there is no look at the table: one barrier, and the slots are safe
// to rewrite after the barriers of the next ticket draw.
template <class V, int W, int U>
__device__ __forceinline__ void exchange_carries_rows(const V (&totA)[U], const V (&totX)[U], V& c, V* slots, int w,
                                                      int lane, int first, V row_start) {
    V TA = totA[0], TX = totX[0];
#pragma unroll
    for (int j = 1; j < U; ++j) {
        TX = vfma(TX, totA[j], totX[j]);
        TA = vmul(TA, totA[j]);
    }
    if (lane == 0) {
        slots[2 * w] = TA;
        slots[2 * w + 1] = TX;
    }
    __syncthreads();
    V runA = vone<V>(), runX = vzero<V>();
    V mineA = runA, mineX = runX;
#pragma unroll
    for (int i = 0; i < W; ++i) {
        const V Ai = slots[2 * i];
        const V Xi = slots[2 * i + 1];
        runA = vselect(i == first, vone<V>(), runA);
        runX = vselect(i == first, vzero<V>(), runX);
        mineA = vselect(i == w, runA, mineA);
        mineX = vselect(i == w, runX, mineX);
        runX = vfma(runX, Ai, Xi);
        runA = vmul(runA, Ai);
    }
    c = vfma(mineA, row_start, mineX);
}
// A wave of such a tile that has no row (the tile's waves are not a multiple of a
// row's, or the rows ran out) keeps the barrier company.
__device__ __forceinline__ void exchange_carries_rows_idle() { __syncthreads(); }

}  // namespace
}  // namespace ascan

#endif  // ASCAN_SPLIT_H_
