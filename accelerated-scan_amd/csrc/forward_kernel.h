// The forward / reverse scan kernel.

#ifndef ASCAN_FORWARD_KERNEL_H_
#define ASCAN_FORWARD_KERNEL_H_

#include <type_traits>

#include "access.h"
#include "carry.h"
#include "gate.h"
#include "packed.h"
#include "split.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Forward kernel (REV = false) and plain reverse scan (REV = true).
// A workgroup holds R rows x W waves per row (R = blockDim.x / 64 / W); the
// rows of a workgroup are adjacent in memory, so with W*R = 16 one tile step
// of the workgroup covers one contiguous span of 16 sub-tiles.
// ---------------------------------------------------------------------------
// SPLIT: kWholeRows, kSweep or kSweepRows (split.h); with kSweepRows `group` is the number of rows a tile holds.
template <class Tr, int W, int U, bool REV, bool ALIGNED, bool REGULAR, int SPLIT, int ACT, bool PACKED>
__global__ void __launch_bounds__(64 * kMaxWavesPerBlock)
    scan_forward_kernel(const typename Tr::S* __restrict__ gates, const typename Tr::TokS* __restrict__ tokens,
                        typename Tr::S* __restrict__ out, int64_t rows, int64_t T, SplitHeader* split,
                        const typename Tr::S* __restrict__ initial, int G, int group) {
    using S = typename Tr::S;
    using V = typename Tr::V;
    constexpr int EPV = Tr::EPV;
    constexpr int64_t SUB = (int64_t)U * 64 * EPV;
    constexpr int64_t TILE = SUB * W;
    static_assert(!PACKED || (!SPLIT && !REGULAR), "packed rows use the general kernels, one group per workgroup");
    constexpr bool ROWS = SPLIT == kSweepRows;

    // Packed rows: this workgroup scans rows [first_row, first_row + nrows) as one row of `len` elements.
    const int64_t first_row = PACKED ? (int64_t)blockIdx.x * group : 0;
    const int64_t len = PACKED ? (rows - first_row < group ? rows - first_row : (int64_t)group) * T : T;
    const int64_t longest = PACKED ? (int64_t)group * T : T;
    // rows start at the same misalignment when their length is a multiple of the grid spacing
    const int head = REGULAR ? 0 : (ALIGNED ? ((longest & (G - 1)) == 0 ? row_lead<Tr>(gates, G) : G - 1) : 0);
    const int64_t ntiles = tiles_per_row(longest, TILE, head);  // 1 when a tile holds several rows
    // Several rows per tile: a row takes as many waves as it has sub-tiles, the tile as many rows as fit.
    const int row_waves = ROWS ? (int)tiles_per_row(longest, SUB, head) : W;
    const int64_t units = ROWS ? (rows + group - 1) / group : rows;  // what the tickets count: rows, or tiles of rows
    __shared__ V slots_all[W == 1 ? 1 : 2 * kSlotsPerBuffer];
    __shared__ S stage_all[PACKED ? W * SUB : 1];
    // Split rows: the workgroups take tiles by ticket, in memory order, until none
    // is left; a workgroup only ever waits for tiles whose owners started before it.
    __shared__ int split_mailbox[4];  // two mailboxes, taken in turn
    __shared__ u32x4_t parked[SPLIT ? 2 * U * 64 : 1];  // wave 0's raw vectors during its walk back
    // Gates with a non-linearity, swept mask-free kernels: what pass 1 made of the stored values waits for pass 2
    // in LDS, each lane's own words (up to 128 KiB per workgroup; the compute unit holds this one workgroup and
    // most of its LDS was free), instead of being evaluated again.  16-bit storage has room for one word per
    // element: the gate, or for the interpolating gate the smaller of gate and complement with the sign of the
    // stored value, from which both come back.  fp32 storage has room for gate and token (KEEP_BOTH), which also
    // frees the registers of the raw vectors, so the normalised exponential gate's kernel takes 4 KiB per wave
    // like the others (forward_split_blocks): (8,1536,T) fp32 forward, ms, T = 65536 / 49152: 1.60 -> 1.50,
    // 1.35 -> 1.12; interpolating gate 1.52 -> 1.48, sigmoid 1.51 -> 1.49, exponential 1.49 -> 1.48.
    constexpr bool kReal = Tr::kNarrow || std::is_same<S, float>::value;
    constexpr bool KEEP_BOTH = std::is_same<S, float>::value && kGateTakesValues<ACT> && SPLIT != kWholeRows && REGULAR;
    constexpr bool KEEP_LDS = KEEP_BOTH || (kReal && SPLIT != kWholeRows && REGULAR &&
                                            (ACT == kGateSigmoid || ACT == kGateExp || ACT == kGateSigmoidLerp));
    constexpr int NKEEP = KEEP_BOTH ? 2 : 1;
    // complex64, swept mask-free kernel: every wave's raw vectors wait for pass 2 in LDS (128 KiB), not only
    // wave 0's during its look at the table; that is what lets the kernel take 4 KiB per wave (128 registers,
    // no scratch; (8,768,65536) forward swept 2.03 ms with 2 KiB per wave, 1.59 like this, 1.64 on whole rows).
    constexpr bool STAGE_LDS = !kReal && SPLIT == kSweep && REGULAR;
    __shared__ u32x4_t staged[STAGE_LDS ? W * U * 2 * 64 : 1];
    __shared__ f32x4_t kept[KEEP_LDS ? W * U * NKEEP * (EPV / 4) * 64 : 1];
    const unsigned long long split_wait_limit = SPLIT == kSweep ? split->wait_limit : 0ull;  // the longest wait allowed
    int visit_parity = 0;
    for (bool first_visit = true;; first_visit = false, visit_parity ^= 1) {
    int64_t row;
    int w, slot_base;
    int64_t k_begin = 0, k_end = ntiles;
    if constexpr (SPLIT) {
        if (!take_split_tile(split, units, ntiles, row, k_begin, split_mailbox + 2 * visit_parity,
                             SPLIT == kSweep ? band_rows(ntiles) : 0)) {
            break;
        }
        k_end = k_begin + 1;
        int thread = threadIdx.x;
        asm volatile("" : "+v"(thread));  // nothing derived from the wave index is carried from visit to visit
        w = thread >> 6;
        slot_base = 0;
    } else if (!first_visit) {
        break;
    } else if constexpr (PACKED) {
        row = first_row;
        w = threadIdx.x >> 6;
        slot_base = 0;
    } else {
        if (!locate_wave<W>(rows, ntiles, row, w, slot_base)) return;  // wave-uniform
    }
    V* slots = slots_all + (W == 1 ? 0 : slot_base);
    // Several rows per tile: `row` so far is the tile; this wave's row and its place among the row's waves.
    const int wave_in_tile = w;
    if constexpr (ROWS) {
        const int wave = __builtin_amdgcn_readfirstlane(w);
        const int row_in_tile = wave / row_waves;
        row = row * group + row_in_tile;
        w = wave - row_in_tile * row_waves;
        if (row_in_tile >= group || row >= rows) {  // wave-uniform: no row for this wave
            exchange_carries_rows_idle();
            continue;
        }
    }

    int64_t lo = (ALIGNED && !REGULAR) ? row_lead<Tr>(gates + row * T, G) : 0;
    // A row rarely fills its last tile.  Swept by ticket, the tile that holds the remainder should be
    // the first of the row in scan order: it waits for no earlier tile and is done at once, where as
    // the last it would sit out the wait for all the others with next to nothing to do (measured,
    // fp32 (8,1536,65533), five tiles per row: forward 1.72 ms with the remainder last, 1.50 ms first).
    // A scan that runs down the addresses has it first as things are; one that runs up is addressed
    // from further below instead, so that its last tile ends on the grid boundary above the row.
    if constexpr (SPLIT == kSweep && !REV && ALIGNED && !REGULAR) lo += ntiles * TILE - ((lo + len + G - 1) & ~(int64_t)(G - 1));  // G is a power of two
    const int64_t hi = lo + len;
    const S* __restrict__ grow = gates + row * T - lo;
    const typename Tr::TokS* __restrict__ trow = tokens + row * T - lo;
    S* __restrict__ orow = out + row * T - lo;

    // state the row starts from (one element per row; absent = zero); a split
    // row needs it in the tiles of its first look-back window; packed rows take theirs at the cuts
    const bool needs_start = !PACKED && initial != nullptr && (!SPLIT || k_begin < kSplitWindow);
    const V row_start = needs_start ? Tr::load1(initial + row) : vzero<V>();
    V carry = row_start;

    // Position of this wave's sub-tile in tile step k.
    auto sub_tile_base = [&](int64_t k) {
        const int64_t tile = REV ? (ntiles - 1 - k) : k;
        return tile * TILE + (int64_t)(REV ? (row_waves - 1 - w) : w) * SUB;
    };
    // Swept tiles: the state entering this wave's sub-tile, from the totals of the tile's waves and, for
    // a row of several tiles, from the row's earlier tiles (wave 0 sets its vectors aside meanwhile).
    auto hand_over = [&](const V (&totA)[U], const V (&totX)[U], V& c, int64_t k, int lane, auto set_aside,
                         auto take_back) {
        if constexpr (ROWS) {
            exchange_carries_rows<V, W, U>(totA, totX, c, slots, wave_in_tile, lane, wave_in_tile - w, row_start);
        } else {
            exchange_carries_split<V, W, U, true>(totA, totX, c, slots, w, lane, split, split_wait_limit,
                                            split_records(split) + row * ntiles, k, ntiles, row_start, set_aside,
                                            take_back);
        }
    };
    // One tile step of this wave.  FULL (a compile-time flag) says that the
    // wave's sub-tile lies entirely inside the row: that copy of the body has no
    // masking code.  The other copy serves the (at most two) ragged tiles of a
    // row; it exists only in the kernels for arbitrary row starts and lengths.
    auto tile_step = [&](int64_t k, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        // The ragged copy (at most two tile steps of a row) works out whatever depends
        // on the lane on the spot: made opaque here, none of it is computed ahead of
        // the tile loop and kept in registers (or scratch) through the mask-free copy.
        int lane = threadIdx.x & 63;
        if constexpr (!FULL || SPLIT) asm volatile("" : "+v"(lane));  // split rows: one tile step per visit, same reasoning
        const int64_t sub_base = sub_tile_base(k);
        const Window win = make_window(lo, hi, sub_base);
        const bool touches = FULL || (win.hi > 0 && win.lo < SUB);  // wave-uniform
        const S* __restrict__ gsub = grow + sub_base;
        const typename Tr::TokS* __restrict__ tsub = trow + sub_base;
        S* __restrict__ osub = orow + sub_base;

        Cuts<Tr> cuts;
        if constexpr (PACKED) {
            cuts = stage_row_starts<Tr>(initial != nullptr ? initial + first_row : nullptr, (int)T, (int)len,
                                        (int)(sub_base - lo), (int)SUB, stage_all + w * SUB, lane);
        }

        // A sub-tile that holds nothing of the row (the waves past the row's end in its last
        // tile step) contributes the identity to the scan: the wave passes the carry on and
        // is done, instead of running both passes over filler values.  With one workgroup per
        // compute unit that arithmetic is not hidden: four waves share a SIMD, and a tile step
        // that moves a few elements would still cost the vector ALU time of a full one.
        if constexpr (!FULL && !SPLIT) {
            if (!touches) {  // wave-uniform
                V totA[U], totX[U];
#pragma unroll
                for (int j = 0; j < U; ++j) {
                    totA[j] = vone<V>();
                    totX[j] = vzero<V>();
                }
                V c;
                exchange_carries<V, W, U, PACKED>(totA, totX, carry, c, slots, (int)(k & 1), w, lane);
                return;
            }
        }

        // (split rows: the same, and the wave still takes its part in the hand-over between tiles)
        if constexpr (!FULL && SPLIT) {
            if (!touches) {  // wave-uniform
                V totA[U], totX[U];
#pragma unroll
                for (int j = 0; j < U; ++j) {
                    totA[j] = vone<V>();
                    totX[j] = vzero<V>();
                }
                V c;
                hand_over(totA, totX, c, k, lane, [] {}, [] {});
                return;
            }
        }

        u32x4_t graw[U], traw[U];
        if (touches) {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int off = vec_offset<U, EPV, REV>(j, lane);
                graw[j] = load_raw<Tr, ALIGNED, FULL>(gsub, off, win, identity_gate<ACT, V>());
                traw[j] = load_tok_raw<Tr, ALIGNED, FULL>(tsub, off, win, vzero<V>());
            }
        } else {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                graw[j] = fill_raw<Tr>(identity_gate<ACT, V>());
                traw[j] = fill_raw<Tr>(vzero<V>());
            }
        }

        // Pass 1: fold each vector into one (A, X) pair and scan the pairs.
        V totA[U], totX[U], exA[U], exX[U];
        CutAt<V> cut_found[PACKED ? U : 1];  // packed rows: where each vector is cut, kept for pass 2
        // 16-bit storage with a gate non-linearity: eight exponentials and reciprocals per vector and
        // pass make the vector ALU the limit (about 5.4 TB/s for the interpolating gate), so the
        // activated gates and tokens of pass 1 are kept for pass 2; the raw vectors are dead by then.
        // The swept kernels have no registers for that (wave 0 parks only its raw vectors), and one workgroup
        // per compute unit hides none of the arithmetic: the mask-free ones keep a word per element in LDS
        // (KEEP_LDS above; measured, bf16 / fp16 (8,1536,65536), ms: sigmoid 0.92 / 0.89 -> 0.75 / 0.73,
        // against 0.79 on whole rows, and 0.76 / 0.74 with the gates kept in registers; exponential
        // 0.83 / 0.81 -> 0.75 / 0.75; interpolating gate 0.96 / 0.98 -> 0.86 / 0.89, whole rows 0.80), except
        // the normalised exponential gate's, which needs gate and token, has 2 KiB per wave and keeps both
        // in registers (1.23 -> 0.94, 0.98 through LDS; whole rows 0.81).
        // Everywhere else unpacking again is cheaper than the registers (the kernels would spill).
        constexpr bool KEEP = Tr::kNarrow && ACT != kGateIdentity && !PACKED &&
                              (!SPLIT || (SPLIT == kSweep && REGULAR && ACT == kGateExpNorm && !KEEP_LDS));
        V gkeep[KEEP ? U : 1][EPV], tkeep[KEEP ? U : 1][EPV];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            V g[EPV], t[EPV];
            Tr::unpack(graw[j], g);
            Tr::unpack(traw[j], t);
            if constexpr (KEEP_LDS) {
                V word[EPV];
                if constexpr (ACT == kGateSigmoidLerp && !KEEP_BOTH) {
#pragma unroll
                    for (int e = 0; e < EPV; ++e) {
                        float gate, complement;
                        word[e] = sigmoid_pair_kept(g[e], gate, complement);
                        g[e] = gate;
                        t[e] = complement * t[e];
                    }
                } else {
                    activate_pair<ACT>(g, t);
#pragma unroll
                    for (int e = 0; e < EPV; ++e) word[e] = g[e];
                }
                f32x4_t* mine = kept + (wave_in_tile * U + j) * (NKEEP * (EPV / 4) * 64) + lane;
#pragma unroll
                for (int h = 0; h < EPV / 4; ++h) {
                    mine[h * 64] = f32x4_t{word[4 * h], word[4 * h + 1], word[4 * h + 2], word[4 * h + 3]};
                    if constexpr (KEEP_BOTH) {
                        mine[(EPV / 4 + h) * 64] = f32x4_t{t[4 * h], t[4 * h + 1], t[4 * h + 2], t[4 * h + 3]};
                    }
                }
            } else {
                activate_pair<ACT>(g, t);
            }
            if constexpr (KEEP) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    gkeep[j][e] = g[e];
                    tkeep[j][e] = t[e];
                }
            }
            if constexpr (PACKED) {
                const int rel = (int)(sub_base - lo) + vec_offset<U, EPV, REV>(j, lane);
                cut_found[j] = locate_cut<Tr, REV>(rel, cuts);
                cut_rows<Tr, REV>(g, t, rel, cuts, cut_found[j]);
            }
            constexpr int e0 = REV ? EPV - 1 : 0;
            V A = g[e0];
            V X = t[e0];
#pragma unroll
            for (int i = 1; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                X = carry_in<PACKED>(g[e], X, t[e]);
                A = gate_product<PACKED>(A, g[e]);
            }
            wave_scan_inclusive<PACKED>(A, X);
            totA[j] = read_lane<63>(A);
            totX[j] = read_lane<63>(X);
            exA[j] = shift_up1(A, vone<V>());
            exX[j] = shift_up1(X, vzero<V>());
            if constexpr (STAGE_LDS) {
                staged[((wave_in_tile * U + j) * 2) * 64 + lane] = graw[j];
                staged[((wave_in_tile * U + j) * 2 + 1) * 64 + lane] = traw[j];
            }
        }

        V c;
        if constexpr (SPLIT) {
            hand_over(
                totA, totX, c, k, lane,
                [&] {
                    if constexpr (!STAGE_LDS) {
#pragma unroll
                        for (int j = 0; j < U; ++j) {
                            parked[(2 * j) * 64 + lane] = graw[j];
                            parked[(2 * j + 1) * 64 + lane] = traw[j];
                        }
                    }
                },
                [&] {
                    if constexpr (!STAGE_LDS) {
#pragma unroll
                        for (int j = 0; j < U; ++j) {
                            graw[j] = parked[(2 * j) * 64 + lane];
                            traw[j] = parked[(2 * j + 1) * 64 + lane];
                        }
                    }
                });
        } else {
            exchange_carries<V, W, U, PACKED>(totA, totX, carry, c, slots, (int)(k & 1), w, lane);
        }

        // Pass 2: the plain recurrence from the state entering each lane.
#pragma unroll
        for (int j = 0; j < U; ++j) {
            V g[EPV], t[EPV];
            if constexpr (KEEP) {
#pragma unroll
                for (int e = 0; e < EPV; ++e) {
                    g[e] = gkeep[j][e];
                    t[e] = tkeep[j][e];
                }
            } else if constexpr (KEEP_LDS) {
                if constexpr (!KEEP_BOTH) {
                    forget_unpacked(traw[j]);
                    Tr::unpack(traw[j], t);
                }
                const f32x4_t* mine = kept + (wave_in_tile * U + j) * (NKEEP * (EPV / 4) * 64) + lane;
#pragma unroll
                for (int h = 0; h < EPV / 4; ++h) {
                    const f32x4_t word = mine[h * 64];
                    g[4 * h] = word.x, g[4 * h + 1] = word.y, g[4 * h + 2] = word.z, g[4 * h + 3] = word.w;
                    if constexpr (KEEP_BOTH) {
                        const f32x4_t tok = mine[(EPV / 4 + h) * 64];
                        t[4 * h] = tok.x, t[4 * h + 1] = tok.y, t[4 * h + 2] = tok.z, t[4 * h + 3] = tok.w;
                    }
                }
                if constexpr (ACT == kGateSigmoidLerp && !KEEP_BOTH) {
#pragma unroll
                    for (int e = 0; e < EPV; ++e) {
                        float gate, complement;
                        sigmoid_pair_from_kept(g[e], gate, complement);
                        g[e] = gate;
                        t[e] = complement * t[e];
                    }
                }
            } else {
                if constexpr (STAGE_LDS) {
                    graw[j] = staged[((wave_in_tile * U + j) * 2) * 64 + lane];
                    traw[j] = staged[((wave_in_tile * U + j) * 2 + 1) * 64 + lane];
                }
                if constexpr (Tr::kNarrow) {
                    forget_unpacked(graw[j]);
                    forget_unpacked(traw[j]);
                }
                Tr::unpack(graw[j], g);
                Tr::unpack(traw[j], t);
                activate_pair<ACT>(g, t);
            }
            if constexpr (PACKED) {
                cut_rows<Tr, REV>(g, t, (int)(sub_base - lo) + vec_offset<U, EPV, REV>(j, lane), cuts, cut_found[j]);
            }
            V x = carry_in<PACKED>(exA[j], c, exX[j]);  // state entering this lane's vector
            c = carry_in<PACKED>(totA[j], c, totX[j]);  // state entering the next block
            V o[EPV];
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                x = carry_in<PACKED>(g[e], x, t[e]);
                o[e] = x;
            }
            const int off = vec_offset<U, EPV, REV>(j, lane);
            if (touches) store_vec<Tr, ALIGNED, FULL>(osub, off, win, o);
        }
    };

    // (Issuing the loads of step k+1 before the arithmetic of step k was tried
    // and measured no faster: the memory system is already saturated by the
    // other workgroups.)
    for (int64_t k = k_begin; k < k_end; ++k) {
        if constexpr (REGULAR) {
            tile_step(k, std::true_type{});
        } else {
            const int64_t sub_base = sub_tile_base(k);
            if (sub_base >= lo && sub_base + SUB <= hi) {  // wave-uniform
                tile_step(k, std::true_type{});
            } else {
                tile_step(k, std::false_type{});
            }
        }
    }
    }  // visits
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_FORWARD_KERNEL_H_
