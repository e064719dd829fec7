// The fused backward kernel.

#ifndef ASCAN_BACKWARD_KERNEL_H_
#define ASCAN_BACKWARD_KERNEL_H_

#include <type_traits>

#include "access.h"
#include "carry.h"
#include "gate.h"
#include "packed.h"
#include "split.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Fused backward kernel: reverse-time scan over gate[t+1] producing d_tokens,
// and d_gates[t] = d_tokens[t] * conj(x[t-1]) in the same pass.
// REV says which way the kernel's scan runs through memory.  REV = true is the
// case above, the backward pass of a forward-time scan: the gradient scan runs
// down the addresses.  REV = false is its mirror image, the backward pass of a
// reverse scan x[t] = gate[t] x[t+1] + token[t]: g[t] = grad_out[t] + conj(gate[t-1]) g[t-1]
// runs up the addresses and d_gates[t] = g[t] conj(x[t+1]).  Below, "after" and
// "before" are meant in the order of the scan being differentiated.
// With the interpolating gate (x[t] = a x[t-1] + (1 - a) v[t], a = sigmoid(z))
// the kernel also reads the values v and writes, for the same g,
// d_v[t] = g[t] (1 - a[t]) and d_z[t] = g[t] (x[t-1] - v[t]) a[t] (1 - a[t]); with the
// normalised exponential gate (x[t] = a x[t-1] + b v[t], a = exp(z), b = sqrt(1 - a^2))
// d_v[t] = g[t] b[t] and d_z[t] = g[t] (a[t] x[t-1] - v[t] a[t]^2 / b[t]).
// ---------------------------------------------------------------------------
// SPLIT: kWholeRows, kSweep or kSweepRows (split.h); with kSweepRows `group` is the number of rows a tile holds.
template <class Tr, int W, int U, bool REV, bool ALIGNED, bool REGULAR, int SPLIT, int ACT, bool PACKED>
__global__ void __launch_bounds__(64 * kMaxWavesPerBlock)
    scan_backward_kernel(const typename Tr::S* __restrict__ gates, const typename Tr::S* __restrict__ states,
                         const typename Tr::S* __restrict__ grad_out, typename Tr::S* __restrict__ d_gates,
                         typename Tr::TokS* __restrict__ d_tokens, int64_t rows, int64_t T, SplitHeader* split,
                         const typename Tr::S* __restrict__ initial, typename Tr::S* __restrict__ d_initial, int G,
                         int group, const typename Tr::S* __restrict__ values) {
    using S = typename Tr::S;
    using V = typename Tr::V;
    constexpr int EPV = Tr::EPV;
    constexpr int64_t SUB = (int64_t)U * 64 * EPV;
    constexpr int64_t TILE = SUB * W;
    static_assert(!PACKED || (!SPLIT && !REGULAR), "packed rows use the general kernels, one group per workgroup");
    static_assert(REV || ACT == kGateIdentity, "the gated scans run forward in time only");
    constexpr bool ROWS = SPLIT == kSweepRows;
    constexpr bool LERP = kGateTakesValues<ACT>;  // `values` is a fourth input
    // index, inside a vector, of the element the gradient scan reaches first / last
    constexpr int E_FIRST = REV ? Tr::EPV - 1 : 0;
    constexpr int E_LAST = REV ? 0 : Tr::EPV - 1;
    constexpr int NIN = LERP ? 4 : 3;
    // The states (and the values of a gate with values) are needed by pass 2 only.  Requested after pass 1,
    // they travel while the tile looks at the table -- about 3 us under load in which nothing else of this
    // compute unit's is in flight -- and wave 0, which does the looking, leaves them in flight into their
    // registers instead of setting them aside with the rest.  The compiler orders the loads that way, or
    // halfway through pass 1, in most swept instantiations by itself; where it does not, holding them back
    // by hand pays, and where it does, the hand-made order is the worse one.  Measured, backward kernel,
    // ms, compiler's order -> states held back, (8,1536,T) unless said otherwise:
    //   fp32, rows of any start and length: reverse scans (all twelve loads were up front, and the kernel
    //   trailed its mirror image by 3.4 %) T = 65533 2.53 -> 2.44, 50001 2.01 -> 1.90, 20000 0.885 -> 0.785;
    //   forward scans 2.45 -> 2.43, 1.89 -> 1.89, 0.783 -> 0.787, 12000 0.467 -> 0.456;
    //   fp32 mask-free, gates with values (half of a tile's reads): interpolating gate 3.11 -> 2.89,
    //   normalised exponential gate 3.23 -> 2.93; with masking code 50001 2.42 -> 2.34 but 20000 0.93 -> 1.00;
    //   fp32 mask-free, identity 2.437 -> 2.448, sigmoid and exponential gate 2.46 -> 2.53;
    //   bf16 / fp16 mask-free: identity 1.240 -> 1.239, exponential gate 1.31 -> 1.25 (fp16 the same), and
    //   the sigmoid and the interpolating gate, which lost when swept before, now gain on whole rows per
    //   workgroup (1.46 -> 1.33, 1.73 -> 1.59); with masking code T = 65533 identity 1.38 -> 1.43;
    //   complex64 (1,16,524288) 0.081 -> 0.075, (1,16,500001) 0.087 -> 0.085, (1,3,4000000) 0.118 -> 0.112.
    // So the switch is on for the classes that gain.  The kernels that own whole rows never hold loads
    // back: nothing to wait for follows pass 1 (bf16 (8,1536,12000) 0.26 -> 0.31 ms when they did).
    constexpr bool kReal32 = !Tr::kNarrow && std::is_same<V, float>::value;
    constexpr bool STATES_LATE =
        SPLIT == kSweep && (kReal32       ? (!REGULAR && ACT == kGateIdentity) || (REGULAR && LERP)
                            : Tr::kNarrow ? REGULAR && ACT != kGateIdentity
                                          : true);

    const int lane = threadIdx.x & 63;
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
    __shared__ u32x4_t parked[SPLIT ? NIN * U * 64 : 1];  // wave 0's raw vectors during its walk back
    __shared__ V parked_values[SPLIT ? 4 * U * 64 : 1];  // and its per-lane scan results
    // 16-bit gates, 16-wave workgroups: what pass 1 made of the stored gates -- the gate and, for a gate with
    // values, the factor of the values -- waits for pass 2 in LDS, each lane's own words (128 KiB per workgroup),
    // instead of being evaluated again.  The compute unit holds this one workgroup (its registers allow no
    // second), nothing else covers its vector ALU time, its registers are taken, and nine tenths of its LDS
    // were free.  Measured, bf16 (8,1536,65536) backward, ms, swept kernels: sigmoid 1.34 -> 1.24, interpolating
    // gate 1.58 -> 1.45, exponential 1.26 -> 1.24, normalised exponential 1.72 -> 1.49; fp16 alike.  With
    // masking code (T = 65533), swept: sigmoid 1.62 -> 1.39, whole rows: 1.53 -> 1.49, interpolating gate
    // 1.92 -> 1.82, exponential (swept) 1.47 -> 1.36, normalised exponential 1.93 -> 1.79; T = 40000, whole
    // rows: 0.90 -> 0.89, 1.14 -> 1.10, 0.88 -> 0.89, 1.09 -> 1.08.  The mask-free kernels that own whole rows
    // (calls without a table) are at their register limit with 4 KiB per wave and lose (sigmoid 1.46 -> 1.50
    // with 32 bytes of scratch, exponential 1.44 -> 1.47): they evaluate twice as before.
    // The fp32 kernels have half the arithmetic per byte and gain or lose a per cent, swept and mask-free
    // ((8,1536,T), T = 65536 / 32768, ms: sigmoid 2.49 -> 2.46 / 1.24 -> 1.25, exponential alike, interpolating
    // gate 2.91 -> 2.92 / 1.44 -> 1.45): only the normalised exponential gate's, with a series and a root in
    // its factor, keeps them (2.96 -> 2.93 / 1.46 -> 1.46, T = 49152 2.22 -> 2.19).
    constexpr bool KEEP_LDS =
        ACT != kGateIdentity && W == kMaxWavesPerBlock && !ROWS && !PACKED &&
        (Tr::kNarrow ? SPLIT == kSweep || !REGULAR || kGateTakesValues<ACT>
                     : ACT == kGateExpNorm && SPLIT == kSweep && REGULAR);
    constexpr int NKEEP = kGateTakesValues<ACT> ? 2 : 1;
    __shared__ f32x4_t kept[KEEP_LDS ? W * U * NKEEP * (EPV / 4) * 64 : 1];
    const unsigned long long split_wait_limit = SPLIT == kSweep ? split->wait_limit : 0ull;  // the longest wait allowed
    int visit_parity = 0;
    for (bool first_visit = true;; first_visit = false, visit_parity ^= 1) {
    int64_t row;
    int w, slot_base;
    int64_t k_begin = 0, k_end = ntiles;
    if constexpr (SPLIT) {
        if (!take_split_tile(split, units, ntiles, row, k_begin, split_mailbox + 2 * visit_parity)) break;
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
    const S* __restrict__ arow = gates + row * T - lo;
    const S* __restrict__ xrow = states + row * T - lo;
    const S* __restrict__ drow = grad_out + row * T - lo;
    const S* __restrict__ vrow = LERP ? values + row * T - lo : nullptr;
    S* __restrict__ dgrow = d_gates + row * T - lo;
    typename Tr::TokS* __restrict__ dtrow = d_tokens + row * T - lo;

    V carry = vzero<V>();
    // the row's index as a scalar (rows < 2^31), for the two per-row addresses
    // below: kept per lane they would sit in vector registers across the tile loop
    const int64_t row_scalar = (int64_t)__builtin_amdgcn_readfirstlane((int)row);

    // Gradient of the state the differentiated scan started from (x[-1]; x[T] for a
    // reverse scan), conj(gate) * g at the row's first (last) element, from g at the
    // position where the gradient scan ends: position 0 of the row's first tile (the
    // top of its last tile).  Positions outside the row carry gate 1 and grad_out 0,
    // and the first of them past the row's end takes the row's outermost gate as the
    // gate that "follows" it -- inside the sub-tile that holds that end.  So if that
    // sub-tile goes on beyond the row, g already is the gradient when it leaves it;
    // with the row flush against the sub-tile's edge the last factor is still missing
    // (sub-tiles that hold nothing of the row are the identity, see a_edge below).
    auto store_start_gradient = [&](V g_end) {
        if (REV ? lo == 0 : hi % SUB == 0) {
            g_end = vmul(vconj(activate1<ACT>(Tr::load1(arow + (REV ? 0 : hi - 1)))), g_end);
        }
        if (lane == 0) Tr::store1(d_initial + row_scalar, g_end);
    };

    // Position of this wave's sub-tile in tile step k of the gradient scan.
    auto sub_tile_base = [&](int64_t k) {
        const int64_t tile = REV ? ntiles - 1 - k : k;
        return tile * TILE + (int64_t)(REV ? row_waves - 1 - w : w) * SUB;
    };
    // Swept tiles: the gradient entering this wave's sub-tile, from the totals of the tile's waves and, for
    // a row of several tiles, from the row's earlier tiles (wave 0 sets its vectors aside meanwhile).
    auto hand_over = [&](const V (&totA)[U], const V (&totX)[U], V& c, int64_t k, int lane, auto set_aside,
                         auto take_back) {
        if constexpr (ROWS) {
            exchange_carries_rows<V, W, U>(totA, totX, c, slots, wave_in_tile, lane, wave_in_tile - w, vzero<V>());
        } else {
            exchange_carries_split<V, W, U, !std::is_same<V, float>::value>(totA, totX, c, slots, w, lane, split, split_wait_limit,
                                            split_records(split) + row * ntiles, k, ntiles, vzero<V>(), set_aside,
                                            take_back);
        }
    };
    // One tile step of this wave; FULL as in the forward kernel.
    auto tile_step = [&](int64_t k, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        // The ragged copy (at most two tile steps of a row) works out whatever depends
        // on the lane on the spot: made opaque here, none of it is computed ahead of
        // the tile loop and kept in registers (or scratch) through the mask-free copy.
        int lane = threadIdx.x & 63;
        if constexpr (!FULL || SPLIT) asm volatile("" : "+v"(lane));  // split rows: one tile step per visit, same reasoning
        const int64_t sub_base = sub_tile_base(k);
        const int64_t sub_end = sub_base + SUB;
        const Window win = make_window(lo, hi, sub_base);
        const bool touches = FULL || (win.hi > 0 && win.lo < SUB);  // wave-uniform
        const S* __restrict__ asub = arow + sub_base;
        const S* __restrict__ dsub = drow + sub_base;
        const S* __restrict__ xsub = xrow + sub_base;
        const S* __restrict__ vsub = LERP ? vrow + sub_base : nullptr;
        S* __restrict__ dgsub = dgrow + sub_base;
        typename Tr::TokS* __restrict__ dtsub = dtrow + sub_base;

        // the state the differentiated scan started from (absent = zero) is needed by
        // the sub-tile that holds the row's first element (last, for a reverse scan)
        V x_start = vzero<V>();
        const int64_t start_at = REV ? lo : hi - 1;
        if (!PACKED && initial != nullptr && sub_base <= start_at && start_at < sub_end) x_start = Tr::load1(initial + row_scalar);  // wave-uniform
        Cuts<Tr> cuts;  // packed rows take their initial states at the cuts instead
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
                // the gradient scan passes through an empty sub-tile unchanged
                if (d_initial != nullptr && k == ntiles - 1 && w == row_waves - 1) store_start_gradient(c);  // wave-uniform
                return;
            }
        }

        u32x4_t araw[U], draw[U], xraw[U], vraw[LERP ? U : 1];
        if (touches) {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int off = vec_offset<U, EPV, REV>(j, lane);
                araw[j] = load_raw<Tr, ALIGNED, FULL>(asub, off, win, identity_gate<ACT, V>());
                draw[j] = load_raw<Tr, ALIGNED, FULL>(dsub, off, win, vzero<V>());
                if constexpr (STATES_LATE) {
                    xraw[j] = fill_raw<Tr>(x_start);  // stands in until the load below
                } else {
                    xraw[j] = load_raw<Tr, ALIGNED, FULL>(xsub, off, win, x_start);
                }
                if constexpr (LERP && STATES_LATE) {
                    vraw[j] = fill_raw<Tr>(vzero<V>());
                } else if constexpr (LERP) {
                    vraw[j] = load_raw<Tr, ALIGNED, FULL>(vsub, off, win, vzero<V>());
                }
            }
        } else {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                araw[j] = fill_raw<Tr>(identity_gate<ACT, V>());
                draw[j] = fill_raw<Tr>(vzero<V>());
                xraw[j] = fill_raw<Tr>(x_start);
                if constexpr (LERP) vraw[j] = fill_raw<Tr>(vzero<V>());
            }
        }

        // The two elements just outside the sub-tile: the gate where the gradient
        // scan comes from (sub_end; sub_base-1 when it runs upwards) and x where it
        // goes next (sub_base-1; sub_end).  Addresses are clamped into the row so the
        // loads are unconditional; out-of-row positions take the identity gate and
        // the state the differentiated scan started from.
        V a_edge, x_edge;
        {
            const int64_t pa = REV ? sub_end : sub_base - 1;
            const int64_t px = REV ? sub_base - 1 : sub_end;
            const int64_t ia = pa < lo ? lo : (pa < hi ? pa : hi - 1);
            const int64_t ix = px < lo ? lo : (px < hi ? px : hi - 1);
            const V av = activate1<ACT>(Tr::load1(arow + ia));
            const V xv = Tr::load1(xrow + ix);
            a_edge = vselect(touches && pa >= lo && pa < hi, av, vone<V>());
            x_edge = vselect(px >= lo && px < hi, xv, x_start);
        }

        // Pass 1.  Gates are needed one element later (gate[t+1]) and states one
        // element earlier (x[t-1]) in the order of the differentiated scan.  The
        // gradient scan runs the other way: the vector it visited just before this
        // lane's belongs to lane-1 and the one it visits next to lane+1, so each
        // block needs one value from each neighbour: a_next (the nearest gate of the
        // vector visited before) and x_prev (the nearest state of the vector visited
        // next).
        V a_next[U], x_prev[U];
        V totA[U], totX[U], exA[U], exX[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            V a[EPV], d[EPV], x[EPV], a_rest[EPV];  // a_rest = 1 - a, interpolating gate only
            Tr::unpack(araw[j], a);
            activate_with_complement<ACT>(a, a_rest);
            if constexpr (KEEP_LDS) {
                f32x4_t* mine = kept + (w * U + j) * (NKEEP * (EPV / 4) * 64) + lane;
#pragma unroll
                for (int h = 0; h < EPV / 4; ++h) {
                    mine[h * 64] = f32x4_t{a[4 * h], a[4 * h + 1], a[4 * h + 2], a[4 * h + 3]};
                    if constexpr (NKEEP == 2) {
                        mine[(EPV / 4 + h) * 64] =
                            f32x4_t{a_rest[4 * h], a_rest[4 * h + 1], a_rest[4 * h + 2], a_rest[4 * h + 3]};
                    }
                }
            }
            Tr::unpack(draw[j], d);
            Tr::unpack(xraw[j], x);
            V hi_edge, lo_edge;
            if (j == 0) {
                hi_edge = a_edge;
            } else {
                V above[EPV];
                Tr::unpack(araw[j > 0 ? j - 1 : 0], above);
                hi_edge = read_lane<63>(activate1<ACT>(above[E_LAST]));
            }
            if (j == U - 1) {
                lo_edge = x_edge;
            } else {
                V below[EPV];
                Tr::unpack(xraw[j < U - 1 ? j + 1 : j], below);
                lo_edge = read_lane<0>(below[E_FIRST]);
            }
            a_next[j] = shift_up1(a[E_LAST], hi_edge);
            x_prev[j] = shift_down1(x[E_FIRST], lo_edge);

            // after[e]: the gate that follows element e; before[e]: the state that precedes it
            V after[EPV], before[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                if constexpr (REV) {
                    after[e] = e < EPV - 1 ? a[e + 1] : a_next[j];
                    before[e] = e > 0 ? x[e - 1] : x_prev[j];
                } else {
                    after[e] = e > 0 ? a[e - 1] : a_next[j];
                    before[e] = e < EPV - 1 ? x[e + 1] : x_prev[j];
                }
            }
            if constexpr (PACKED) {
                bool is_first[EPV];
                int row_of[EPV];
                cut_rows_backward<Tr, REV>(after, before, is_first, row_of,
                                           (int)(sub_base - lo) + vec_offset<U, EPV, REV>(j, lane), cuts);
            }
            V A = vconj(after[E_FIRST]);
            V X = d[E_FIRST];
#pragma unroll
            for (int i = 1; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                const V ga = vconj(after[e]);
                X = carry_in<PACKED>(ga, X, d[e]);
                A = gate_product<PACKED>(A, ga);
            }
            wave_scan_inclusive<PACKED>(A, X);
            totA[j] = read_lane<63>(A);
            totX[j] = read_lane<63>(X);
            exA[j] = shift_up1(A, vone<V>());
            exX[j] = shift_up1(X, vzero<V>());
        }

        if constexpr (STATES_LATE) {
            // the offset waits for pass 1's last total, so the loads cannot be moved ahead of it
            const int late = zero_after(totX[U - 1]);
            if (touches) {
#pragma unroll
                for (int j = 0; j < U; ++j) {
                    xraw[j] = load_raw<Tr, ALIGNED, FULL>(xsub, vec_offset<U, EPV, REV>(j, lane) + late, win, x_start);
                    if constexpr (LERP) {
                        vraw[j] = load_raw<Tr, ALIGNED, FULL>(vsub, vec_offset<U, EPV, REV>(j, lane) + late, win, vzero<V>());
                    }
                }
            }
        }

        V c;
        if constexpr (SPLIT) {
            hand_over(
                totA, totX, c, k, lane,
                [&] {
#pragma unroll
                    for (int j = 0; j < U; ++j) {
                        parked[(NIN * j) * 64 + lane] = araw[j];
                        parked[(NIN * j + 1) * 64 + lane] = draw[j];
                        if constexpr (!STATES_LATE) {  // late loads stay in flight into their registers
                            parked[(NIN * j + 2) * 64 + lane] = xraw[j];
                            if constexpr (LERP) parked[(NIN * j + 3) * 64 + lane] = vraw[j];
                        }
                        parked_values[(4 * j) * 64 + lane] = a_next[j];
                        parked_values[(4 * j + 1) * 64 + lane] = x_prev[j];
                        parked_values[(4 * j + 2) * 64 + lane] = exA[j];
                        parked_values[(4 * j + 3) * 64 + lane] = exX[j];
                    }
                },
                [&] {
#pragma unroll
                    for (int j = 0; j < U; ++j) {
                        araw[j] = parked[(NIN * j) * 64 + lane];
                        draw[j] = parked[(NIN * j + 1) * 64 + lane];
                        if constexpr (!STATES_LATE) {
                            xraw[j] = parked[(NIN * j + 2) * 64 + lane];
                            if constexpr (LERP) vraw[j] = parked[(NIN * j + 3) * 64 + lane];
                        }
                        a_next[j] = parked_values[(4 * j) * 64 + lane];
                        x_prev[j] = parked_values[(4 * j + 1) * 64 + lane];
                        exA[j] = parked_values[(4 * j + 2) * 64 + lane];
                        exX[j] = parked_values[(4 * j + 3) * 64 + lane];
                    }
                });
        } else {
            exchange_carries<V, W, U, PACKED>(totA, totX, carry, c, slots, (int)(k & 1), w, lane);
        }
        // Pass 2: the plain reverse recurrence and the gate gradient.
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if constexpr (Tr::kNarrow) {
                forget_unpacked(araw[j]);
                forget_unpacked(draw[j]);
                forget_unpacked(xraw[j]);
                if constexpr (LERP) forget_unpacked(vraw[j]);
            }
            V a[EPV], d[EPV], x[EPV], a_rest[EPV], v[LERP ? EPV : 1];
            if constexpr (KEEP_LDS) {
                const f32x4_t* mine = kept + (w * U + j) * (NKEEP * (EPV / 4) * 64) + lane;
#pragma unroll
                for (int h = 0; h < EPV / 4; ++h) {
                    const f32x4_t ka = mine[h * 64];
                    a[4 * h] = ka.x, a[4 * h + 1] = ka.y, a[4 * h + 2] = ka.z, a[4 * h + 3] = ka.w;
                    if constexpr (NKEEP == 2) {
                        const f32x4_t kr = mine[(EPV / 4 + h) * 64];
                        a_rest[4 * h] = kr.x, a_rest[4 * h + 1] = kr.y, a_rest[4 * h + 2] = kr.z, a_rest[4 * h + 3] = kr.w;
                    }
                }
            } else {
                Tr::unpack(araw[j], a);
                activate_with_complement<ACT>(a, a_rest);
            }
            Tr::unpack(draw[j], d);
            Tr::unpack(xraw[j], x);
            if constexpr (LERP) Tr::unpack(vraw[j], v);
            if constexpr (STATES_LATE) {  // pass 1 saw stand-ins
                V lo_edge = x_edge;
                if (j < U - 1) {
                    V below[EPV];
                    Tr::unpack(xraw[j < U - 1 ? j + 1 : j], below);
                    lo_edge = read_lane<0>(below[E_FIRST]);
                }
                x_prev[j] = shift_down1(x[E_FIRST], lo_edge);
            }
            V gr = carry_in<PACKED>(exA[j], c, exX[j]);  // g entering this lane's vector
            c = carry_in<PACKED>(totA[j], c, totX[j]);
            const int off = vec_offset<U, EPV, REV>(j, lane);
            V after[EPV], before[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                if constexpr (REV) {
                    after[e] = e < EPV - 1 ? a[e + 1] : a_next[j];
                    before[e] = e > 0 ? x[e - 1] : x_prev[j];
                } else {
                    after[e] = e > 0 ? a[e - 1] : a_next[j];
                    before[e] = e < EPV - 1 ? x[e + 1] : x_prev[j];
                }
            }
            bool is_first[EPV];
            int row_of[EPV];
            if constexpr (PACKED) {
                cut_rows_backward<Tr, REV>(after, before, is_first, row_of, (int)(sub_base - lo) + off, cuts);
            }
            V dt[EPV], dg[EPV], gs[PACKED ? EPV : 1];  // gs: g itself, for the rows' initial states
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                gr = carry_in<PACKED>(vconj(after[e]), gr, d[e]);
                if constexpr (PACKED) gs[e] = gr;
                if constexpr (ACT == kGateSigmoidLerp) {
                    // token = (1 - a) v:  d_v = g (1 - a);  d_a = g (x[t-1] - v);  d_z = d_a a (1 - a)
                    dt[e] = gr * a_rest[e];
                    dg[e] = (gr * (before[e] - v[e])) * (a[e] * a_rest[e]);
                } else if constexpr (ACT == kGateExpNorm) {
                    // token = b v, b = sqrt(1 - a^2):  d_v = g b;  d_z = g (a x[t-1] + v db/dz),  db/dz = -a^2 / b
                    // (b = 0, a stored logarithm of exactly 0: the unbounded db/dz is taken as 0)
                    dt[e] = gr * a_rest[e];
                    const V slope = a_rest[e] == 0.0f ? 0.0f : a[e] * __builtin_amdgcn_rcpf(a_rest[e]);
                    dg[e] = gr * (a[e] * (before[e] - v[e] * slope));
                } else {
                    dt[e] = gr;
                    dg[e] = vmul(gr, vconj(before[e]));
                    if constexpr (ACT != kGateIdentity) dg[e] = vmul(dg[e], gate_slope<ACT>(a[e]));
                }
            }
            if (touches) {
                store_tok_vec<Tr, ALIGNED, FULL>(dtsub, off, win, dt);
                store_vec<Tr, ALIGNED, FULL>(dgsub, off, win, dg);
            }
            if constexpr (PACKED) {
                // gradient of each row's initial state, conj(gate[0]) * g[0], from the lane that holds the row's start
                if (d_initial != nullptr) {
#pragma unroll
                    for (int e = 0; e < EPV; ++e) {
                        if (is_first[e]) Tr::store1(d_initial + first_row + row_of[e], vmul(vconj(a[e]), gs[e]));
                    }
                }
            }
        }

        // A split row's last tile step ends where the differentiated scan started: after
        // pass 2, c is g at the last position this wave's sub-tile holds in the gradient scan.
        if constexpr (SPLIT) {
            if (d_initial != nullptr && k == ntiles - 1 && w == row_waves - 1) store_start_gradient(c);  // wave-uniform
        }
    };

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
    // after the last tile step the carry is g at the position where the gradient scan ends
    if constexpr (!SPLIT && !PACKED) {
        if (d_initial != nullptr && w == 0) store_start_gradient(carry);  // wave-uniform
    }
    }  // visits
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_BACKWARD_KERNEL_H_
