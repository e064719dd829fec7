// Chooses and launches the forward kernel of a call for one dtype.
#ifndef ASCAN_FORWARD_DISPATCH_H_
#define ASCAN_FORWARD_DISPATCH_H_

#include "forward_kernel.h"
#include "policy.h"

namespace ascan {
namespace {

template <class Tr, int W, bool REV, bool ALIGNED, bool REGULAR, int ACT>
hipError_t launch_forward(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                          int64_t T, int grid, int rows_per_block, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? Tuning<Tr>::U : Tuning<Tr>::UG;
    const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
    const unsigned threads = 64u * W * rows_per_block;
    return launch(scan_forward_kernel<Tr, W, U, REV, ALIGNED, REGULAR, kWholeRows, ACT, false>, blocks, threads, stream,
                  static_cast<const S*>(gates), static_cast<const TokS*>(tokens), static_cast<S*>(out), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial), grid, 0);
}

// MODE = kSweep: `ntiles` tiles per row; kSweepRows: `rows_per_tile` rows per tile (the table is the ticket alone).
template <class Tr, bool REV, bool REGULAR, int ACT, int MODE>
hipError_t launch_forward_split(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                                int64_t T, int grid, int64_t ntiles, int rows_per_tile, const Workspace& ws,
                                hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = forward_split_blocks<Tr, ACT, REGULAR>(REGULAR ? SplitTuning<Tr>::U : SplitTuning<Tr>::UG);
    auto kernel = scan_forward_kernel<Tr, kSplitWaves, U, REV, true, REGULAR, MODE, ACT, false>;
    // one workgroup per compute unit: the mask-free kernels would fit twice since their waves fold the tile's
    // totals in one row of lanes (63-75 registers), and run no faster that way (fp32 / bf16 (8,1536,65536)
    // 1.483 / 0.735 ms with two, 1.480 / 0.732 with one)
    const unsigned resident = resident_workgroups(kernel, 64 * kSplitWaves, 1);
    if (resident == 0) return hipErrorInvalidConfiguration;
    const bool whole_rows = MODE == kSweepRows;
    const hipError_t e = reset_split_table(ws, whole_rows ? 0 : rows, ntiles, stream);
    if (e != hipSuccess) return e;
    const int64_t tiles = whole_rows ? (rows + rows_per_tile - 1) / rows_per_tile : rows * ntiles;
    return launch(kernel, (unsigned)(tiles < resident ? tiles : resident), 64u * kSplitWaves, stream,
                  static_cast<const S*>(gates), static_cast<const TokS*>(tokens), static_cast<S*>(out), rows, T,
                  static_cast<SplitHeader*>(ws.ptr), static_cast<const S*>(initial), grid, rows_per_tile);
}

template <class Tr, bool REV, bool ALIGNED, int ACT>
hipError_t launch_forward_packed(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                                 int64_t T, int grid, int group, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    const unsigned blocks = (unsigned)((rows + group - 1) / group);
    return launch(scan_forward_kernel<Tr, kPackedWaves, Tuning<Tr>::UG, REV, ALIGNED, false, kWholeRows, ACT, true>, blocks,
                  64u * kPackedWaves, stream, static_cast<const S*>(gates), static_cast<const TokS*>(tokens),
                  static_cast<S*>(out), rows, T, static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial),
                  grid, group);
}

// Turns (gate, reverse, flag) into compile-time tags and calls go(rev, flag, gate).
// A gate other than the identity implies forward time.
template <class Tr, class Go>
hipError_t dispatch_forward(int act, bool reverse, bool flag, Go&& go) {
    return with_gate<Tr>(act, [&](auto gate) {
        constexpr int ACT = decltype(gate)::value;
        if constexpr (ACT != kGateIdentity) {
            return flag ? go(std::false_type{}, std::true_type{}, gate) : go(std::false_type{}, std::false_type{}, gate);
        } else {
            if (reverse) {
                return flag ? go(std::true_type{}, std::true_type{}, gate) : go(std::true_type{}, std::false_type{}, gate);
            }
            return flag ? go(std::false_type{}, std::true_type{}, gate) : go(std::false_type{}, std::false_type{}, gate);
        }
    });
}

template <class Tr>
int forward_typed(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows, int64_t T,
                  bool reverse, int act, const Workspace& ws, hipStream_t stream) {
    constexpr int64_t kElem = (int64_t)sizeof(typename Tr::S);
    constexpr int64_t SUB = (int64_t)Tuning<Tr>::U * 64 * Tr::EPV;    // regular kernels
    constexpr int64_t SUBG = (int64_t)Tuning<Tr>::UG * 64 * Tr::EPV;  // kernels with masking code
    // gates that form the token from values as well do more arithmetic per byte and, like the 16-bit kernels,
    // gain from a narrower plan when the last tile step would be mostly empty
    const bool trim = kTrimPlan<Tr> || gate_takes_values(act);
    Plan plan = choose_plan(T, SUB, kElem, trim);
    const void* const state_like[] = {gates, out};
    const Lead at = find_lead<Tr>(state_like, tokens);
    const bool same_lead = at.same;
    const int lead = at.lead;
    const Access access = choose_access(same_lead, lead, T, SUB * plan.waves_per_row);
    if (access != Access::kRegular) plan = choose_plan(T, SUBG, kElem, trim);
    const int R = plan.rows_per_block;
    hipError_t err = hipSuccess;
    // Gated kernels run forward in time only (validated by the entry points); REV below is a
    // compile-time false for them.
    if (const int group = packed_group(rows, T, kElem, SUBG * kPackedWaves, same_lead ? at.grid : 1)) {
        auto go = [&](auto rev, auto aligned, auto gate) {
            return launch_forward_packed<Tr, decltype(rev)::value, decltype(aligned)::value, decltype(gate)::value>(
                gates, tokens, out, initial, rows, T, at.grid, group, stream);
        };
        err = dispatch_forward<Tr>(act, reverse, same_lead, go);
        return launch_status(err);
    }
    if (same_lead && ws.ptr != nullptr) {
        const int64_t SUBS = (int64_t)forward_split_blocks_of<Tr>(act, SplitTuning<Tr>::U, true) * 64 * Tr::EPV;
        const int64_t SUBSG = (int64_t)forward_split_blocks_of<Tr>(act, SplitTuning<Tr>::UG, false) * 64 * Tr::EPV;
        if constexpr (kSweepClass<Tr> != SweepClass::kComplex) {
            // rows of half a tile: two whole rows per swept tile
            const int per_tile = lead == 0 ? sweep_rows_per_tile(kSweepClass<Tr>, rows, T, kElem, SUBS, act) : 0;
            if (per_tile != 0 && workspace_fits(ws, 0, 1)) {
                auto go = [&](auto rev, auto, auto gate) {
                    return launch_forward_split<Tr, decltype(rev)::value, true, decltype(gate)::value, kSweepRows>(
                        gates, tokens, out, initial, rows, T, at.grid, 1, per_tile, ws, stream);
                };
                err = dispatch_forward<Tr>(act, reverse, true, go);
                return launch_status(err);
            }
        }
        const bool regular = lead == 0 && T % (SUBS * kSplitWaves) == 0;
        const int64_t tile = (regular ? SUBS : SUBSG) * kSplitWaves;
        const int64_t ntiles = host_tiles_per_row<Tr>(T, tile, regular, at);
        if (want_split(kSweepClass<Tr>, rows, T * kElem, tile * kElem, ntiles, act, true, regular) && workspace_fits(ws, rows, ntiles)) {
            auto go = [&](auto rev, auto reg, auto gate) {
                return launch_forward_split<Tr, decltype(rev)::value, decltype(reg)::value, decltype(gate)::value,
                                            kSweep>(gates, tokens, out, initial, rows, T, at.grid, ntiles, 0, ws,
                                                    stream);
            };
            err = dispatch_forward<Tr>(act, reverse, regular, go);
            return launch_status(err);
        }
    }
    auto with_waves = [&](auto aligned, auto reg) {
        auto go = [&](auto rev, auto waves, auto gate) {
            return launch_forward<Tr, decltype(waves)::value, decltype(rev)::value, decltype(aligned)::value,
                                  decltype(reg)::value, decltype(gate)::value>(gates, tokens, out, initial, rows, T,
                                                                               at.grid, R, stream);
        };
        auto by_waves = [&](auto rev, auto, auto gate) {
            switch (plan.waves_per_row) {
                case 1: return go(rev, std::integral_constant<int, 1>{}, gate);
                case 2: return go(rev, std::integral_constant<int, 2>{}, gate);
                case 4: return go(rev, std::integral_constant<int, 4>{}, gate);
                case 8: return go(rev, std::integral_constant<int, 8>{}, gate);
                default: return go(rev, std::integral_constant<int, 16>{}, gate);
            }
        };
        return dispatch_forward<Tr>(act, reverse, true, by_waves);
    };
    if (access == Access::kRegular) {
        err = with_waves(std::true_type{}, std::true_type{});
    } else if (access == Access::kVector) {
        err = with_waves(std::true_type{}, std::false_type{});
    } else {
        err = with_waves(std::false_type{}, std::false_type{});
    }
    return launch_status(err);
}

}  // namespace
}  // namespace ascan

// Defines ascan::NAME, the forward entry of one dtype, in the including file.
#define ASCAN_DEFINE_FORWARD(NAME, TRAITS)                                                              \
    int ascan::NAME(const ascan::ForwardCall& c) {                                                      \
        return ascan::forward_typed<ascan::TRAITS>(c.gates, c.tokens, c.out, c.initial, c.rows, c.seqlen, \
                                                   c.reverse, c.gate, c.workspace, c.stream);           \
    }

#endif  // ASCAN_FORWARD_DISPATCH_H_
