// Chooses and launches the backward kernel of a call for one dtype.
#ifndef ASCAN_BACKWARD_DISPATCH_H_
#define ASCAN_BACKWARD_DISPATCH_H_

#include "backward_kernel.h"
#include "policy.h"

namespace ascan {
namespace {

// The arguments every backward launch passes on unchanged.
struct BackwardBuffers {
    const void* gates;
    const void* states;
    const void* grad_out;
    void* d_gates;
    void* d_tokens;
    const void* initial;
    void* d_initial;
    const void* values;  // the fourth input of a gate with values, else null
};

// REV is the backward kernel's own direction: true for the backward pass of a forward-time scan.
template <class Tr, bool REV, int W, bool ALIGNED, bool REGULAR, int ACT>
hipError_t launch_backward(const BackwardBuffers& b, int64_t rows, int64_t T, int grid, int rows_per_block,
                           hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = backward_blocks<ACT>(REGULAR ? Tuning<Tr>::UB : Tuning<Tr>::UBG);
    const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
    const unsigned threads = 64u * W * rows_per_block;
    return launch(scan_backward_kernel<Tr, W, U, REV, ALIGNED, REGULAR, kWholeRows, ACT, false>, blocks, threads, stream,
                  static_cast<const S*>(b.gates), static_cast<const S*>(b.states), static_cast<const S*>(b.grad_out),
                  static_cast<S*>(b.d_gates), static_cast<TokS*>(b.d_tokens), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(b.initial), static_cast<S*>(b.d_initial),
                  grid, 0, static_cast<const S*>(b.values));
}

// MODE = kSweep: `ntiles` tiles per row; kSweepRows: `rows_per_tile` rows per tile (the table is the ticket alone).
template <class Tr, bool REV, bool REGULAR, int ACT, int MODE>
hipError_t launch_backward_split(const BackwardBuffers& b, int64_t rows, int64_t T, int grid, int64_t ntiles,
                                 int rows_per_tile, const Workspace& ws, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = backward_blocks<ACT>(REGULAR ? SplitTuning<Tr>::UB : SplitTuning<Tr>::UBG);
    auto kernel = scan_backward_kernel<Tr, kSplitWaves, U, REV, true, REGULAR, MODE, ACT, false>;
    const unsigned resident = resident_workgroups(kernel, 64 * kSplitWaves, MODE == kSweepRows ? 1 : kMaxWavesPerBlock);
    if (resident == 0) return hipErrorInvalidConfiguration;
    const bool whole_rows = MODE == kSweepRows;
    const hipError_t e = reset_split_table(ws, whole_rows ? 0 : rows, ntiles, stream);
    if (e != hipSuccess) return e;
    const int64_t tiles = whole_rows ? (rows + rows_per_tile - 1) / rows_per_tile : rows * ntiles;
    return launch(kernel, (unsigned)(tiles < resident ? tiles : resident), 64u * kSplitWaves, stream,
                  static_cast<const S*>(b.gates), static_cast<const S*>(b.states), static_cast<const S*>(b.grad_out),
                  static_cast<S*>(b.d_gates), static_cast<TokS*>(b.d_tokens), rows, T,
                  static_cast<SplitHeader*>(ws.ptr), static_cast<const S*>(b.initial), static_cast<S*>(b.d_initial),
                  grid, rows_per_tile, static_cast<const S*>(b.values));
}

template <class Tr, bool REV, int PW, bool ALIGNED, int ACT>
hipError_t launch_backward_packed(const BackwardBuffers& b, int64_t rows, int64_t T, int grid, int group,
                                  hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    const unsigned blocks = (unsigned)((rows + group - 1) / group);
    return launch(scan_backward_kernel<Tr, PW, Tuning<Tr>::UBG, REV, ALIGNED, false, kWholeRows, ACT, true>, blocks,
                  64u * PW, stream, static_cast<const S*>(b.gates), static_cast<const S*>(b.states),
                  static_cast<const S*>(b.grad_out), static_cast<S*>(b.d_gates), static_cast<TokS*>(b.d_tokens), rows,
                  T, static_cast<SplitHeader*>(nullptr), static_cast<const S*>(b.initial),
                  static_cast<S*>(b.d_initial), grid, group, static_cast<const S*>(b.values));
}

template <class Tr, bool REV>
int backward_typed(const BackwardBuffers& b, int64_t rows, int64_t T, int act, const Workspace& ws,
                   hipStream_t stream) {
    constexpr int64_t kElem = (int64_t)sizeof(typename Tr::S);
    const int64_t SUB = (int64_t)backward_blocks_of(act, Tuning<Tr>::UB) * 64 * Tr::EPV;  // regular kernels
    const int64_t SUBG = (int64_t)backward_blocks_of(act, Tuning<Tr>::UBG) * 64 * Tr::EPV;  // kernels with masking code
    const void* const state_like[] = {b.gates, b.states, b.grad_out, b.d_gates, b.values ? b.values : b.gates};
    const Lead at = find_lead<Tr>(state_like, b.d_tokens);
    const bool same_lead = at.same;
    const int lead = at.lead;
    // the interpolating gate's kernels (half-size tiles, a fourth input, more arithmetic per element) gain from a
    // narrower plan for a mostly empty last tile whatever the dtype: fp32 (8,1536,9000) backward 4.9 -> 5.5 TB/s
    const bool trim = kTrimPlan<Tr> || gate_takes_values(act);
    Plan plan = choose_plan(T, SUB, kElem, trim);
    Access access = choose_access(same_lead, lead, T, SUB * plan.waves_per_row);
    if (access != Access::kRegular) plan = choose_plan(T, SUBG, kElem, trim);
    // fp32 rows of exactly 4 KiB: two waves of 2 KiB per row (the kernel with masking code, whose tile steps
    // inside a row are mask-free as well) instead of one wave of 4 KiB -- measured, (8,1536,1024) 5.7 -> 6.06 TB/s,
    // (32,1536,1024) 6.22 -> 6.26, (2,1536,1024) 5.03 -> 4.95
    if (kSweepClass<Tr> == SweepClass::kF32 && access == Access::kRegular && T == SUB && SUBG * 2 == SUB &&
        forced_plan().waves_per_row == 0 && forced_plan().rows_per_block == 0) {
        access = Access::kVector;
        plan = Plan{2, 2};
    }
    const int R = plan.rows_per_block;
    hipError_t err = hipSuccess;
    // 16-bit rows of 512 bytes and more, vectorised flavour, plenty of them: groups of the wider workgroup
    if constexpr (Tr::kNarrow) {
        if (same_lead && T * kElem >= kPackedWideRowBytes) {
            const int group = packed_group(rows, T, kElem, SUBG * kPackedWavesWide, at.grid);
            if (group != 0 && rows / group >= kPackedWideMinGroups) {
                err = with_gate<Tr, REV>(act, [&](auto gate) {
                    return launch_backward_packed<Tr, REV, kPackedWavesWide, true, decltype(gate)::value>(b, rows, T, at.grid,
                                                                                                     group, stream);
                });
                return launch_status(err);
            }
        }
    }
    if (const int group = packed_group(rows, T, kElem, SUBG * kPackedWaves, same_lead ? at.grid : 1)) {
        err = with_gate<Tr, REV>(act, [&](auto gate) {
            constexpr int ACT = decltype(gate)::value;
            return same_lead ? launch_backward_packed<Tr, REV, kPackedWaves, true, ACT>(b, rows, T, at.grid, group, stream)
                             : launch_backward_packed<Tr, REV, kPackedWaves, false, ACT>(b, rows, T, at.grid, group, stream);
        });
        return launch_status(err);
    }
    if (same_lead && ws.ptr != nullptr) {
        const int64_t SUBS = (int64_t)backward_blocks_of(act, SplitTuning<Tr>::UB) * 64 * Tr::EPV;
        const int64_t SUBSG = (int64_t)backward_blocks_of(act, SplitTuning<Tr>::UBG) * 64 * Tr::EPV;
        if constexpr (kSweepClass<Tr> != SweepClass::kComplex) {
            // rows of half a tile: two whole rows per swept tile
            const int per_tile = lead == 0 ? sweep_rows_per_tile(kSweepClass<Tr>, rows, T, kElem, SUBS, act) : 0;
            if (per_tile != 0 && workspace_fits(ws, 0, 1)) {
                err = with_gate<Tr, REV>(act, [&](auto gate) {
                    return launch_backward_split<Tr, REV, true, decltype(gate)::value, kSweepRows>(b, rows, T, at.grid, 1,
                                                                                                 per_tile, ws, stream);
                });
                return launch_status(err);
            }
        }
        const bool regular = lead == 0 && T % (SUBS * kSplitWaves) == 0;
        const int64_t tile = (regular ? SUBS : SUBSG) * kSplitWaves;
        const int64_t ntiles = host_tiles_per_row<Tr>(T, tile, regular, at);
        if (want_split(kSweepClass<Tr>, rows, T * kElem, tile * kElem, ntiles, act, false, regular) && workspace_fits(ws, rows, ntiles)) {
            err = with_gate<Tr, REV>(act, [&](auto gate) {
                constexpr int ACT = decltype(gate)::value;
                return regular ? launch_backward_split<Tr, REV, true, ACT, kSweep>(b, rows, T, at.grid, ntiles, 0, ws, stream)
                               : launch_backward_split<Tr, REV, false, ACT, kSweep>(b, rows, T, at.grid, ntiles, 0, ws, stream);
            });
            return launch_status(err);
        }
    }
    auto with_waves = [&](auto aligned, auto reg) {
        return with_gate<Tr, REV>(act, [&](auto gate) {
            constexpr int ACT = decltype(gate)::value;
            constexpr bool AL = decltype(aligned)::value, REG = decltype(reg)::value;
            switch (plan.waves_per_row) {
                case 1: return launch_backward<Tr, REV, 1, AL, REG, ACT>(b, rows, T, at.grid, R, stream);
                case 2: return launch_backward<Tr, REV, 2, AL, REG, ACT>(b, rows, T, at.grid, R, stream);
                case 4: return launch_backward<Tr, REV, 4, AL, REG, ACT>(b, rows, T, at.grid, R, stream);
                case 8: return launch_backward<Tr, REV, 8, AL, REG, ACT>(b, rows, T, at.grid, R, stream);
                default: return launch_backward<Tr, REV, 16, AL, REG, ACT>(b, rows, T, at.grid, R, stream);
            }
        });
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

// Defines ascan::NAME, the backward entry of one dtype, in the including file;
// REV = true for the backward pass of forward-time scans, false for that of reverse scans.
#define ASCAN_DEFINE_BACKWARD(NAME, TRAITS, REV)                                                                \
    int ascan::NAME(const ascan::BackwardCall& c) {                                                             \
        const ascan::BackwardBuffers b{c.gates, c.states, c.grad_out, c.d_gates, c.d_tokens, c.initial, c.d_initial, \
                                       c.values};                                                               \
        return ascan::backward_typed<ascan::TRAITS, REV>(b, c.rows, c.seqlen, c.gate, c.workspace, c.stream);   \
    }

#endif  // ASCAN_BACKWARD_DISPATCH_H_
