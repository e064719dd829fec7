// Chooses and launches the backward kernel of a call for one dtype.
#ifndef ASCAN_BACKWARD_DISPATCH_H_
#define ASCAN_BACKWARD_DISPATCH_H_

#include "backward_kernel.h"
#include "policy.h"

namespace ascan {
namespace {

template <class Tr, int W, bool ALIGNED, bool REGULAR, int ACT>
hipError_t launch_backward(const void* gates, const void* states, const void* grad_out, void* d_gates,
                           void* d_tokens, const void* initial, void* d_initial, int64_t rows, int64_t T, int grid,
                           int rows_per_block, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? Tuning<Tr>::UB : Tuning<Tr>::UBG;
    const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
    const unsigned threads = 64u * W * rows_per_block;
    return launch(scan_backward_kernel<Tr, W, U, ALIGNED, REGULAR, false, ACT, false>, blocks, threads, stream,
                  static_cast<const S*>(gates), static_cast<const S*>(states), static_cast<const S*>(grad_out),
                  static_cast<S*>(d_gates), static_cast<TokS*>(d_tokens), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial), static_cast<S*>(d_initial), grid, 0);
}

template <class Tr, bool REGULAR, int ACT>
hipError_t launch_backward_split(const void* gates, const void* states, const void* grad_out, void* d_gates,
                                 void* d_tokens, const void* initial, void* d_initial, int64_t rows, int64_t T,
                                 int grid, int64_t ntiles, const Workspace& ws, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? SplitTuning<Tr>::UB : SplitTuning<Tr>::UBG;
    auto kernel = scan_backward_kernel<Tr, kSplitWaves, U, true, REGULAR, true, ACT, false>;
    const unsigned resident = resident_workgroups(kernel, 64 * kSplitWaves);
    if (resident == 0) return hipErrorInvalidConfiguration;
    const hipError_t e = reset_split_table(ws, rows, ntiles, stream);
    if (e != hipSuccess) return e;
    const int64_t tiles = rows * ntiles;
    return launch(kernel, (unsigned)(tiles < resident ? tiles : resident), 64u * kSplitWaves, stream,
                  static_cast<const S*>(gates), static_cast<const S*>(states), static_cast<const S*>(grad_out),
                  static_cast<S*>(d_gates), static_cast<TokS*>(d_tokens), rows, T,
                  static_cast<SplitHeader*>(ws.ptr), static_cast<const S*>(initial), static_cast<S*>(d_initial), grid, 0);
}

template <class Tr, int PW, bool ALIGNED, int ACT>
hipError_t launch_backward_packed(const void* gates, const void* states, const void* grad_out, void* d_gates,
                                  void* d_tokens, const void* initial, void* d_initial, int64_t rows, int64_t T,
                                  int grid, int group, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    const unsigned blocks = (unsigned)((rows + group - 1) / group);
    return launch(scan_backward_kernel<Tr, PW, Tuning<Tr>::UBG, ALIGNED, false, false, ACT, true>, blocks,
                  64u * PW, stream, static_cast<const S*>(gates), static_cast<const S*>(states),
                  static_cast<const S*>(grad_out), static_cast<S*>(d_gates), static_cast<TokS*>(d_tokens), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial), static_cast<S*>(d_initial), grid,
                  group);
}

template <class Tr>
int backward_typed(const void* gates, const void* states, const void* grad_out, void* d_gates, void* d_tokens,
                   const void* initial, void* d_initial, int64_t rows, int64_t T, int act, const Workspace& ws,
                   hipStream_t stream) {
    constexpr int64_t kElem = (int64_t)sizeof(typename Tr::S);
    constexpr int64_t SUB = (int64_t)Tuning<Tr>::UB * 64 * Tr::EPV;    // regular kernels
    constexpr int64_t SUBG = (int64_t)Tuning<Tr>::UBG * 64 * Tr::EPV;  // kernels with masking code
    const void* const state_like[] = {gates, states, grad_out, d_gates};
    const Lead at = find_lead<Tr>(state_like, d_tokens);
    const bool same_lead = at.same;
    const int lead = at.lead;
    Plan plan = choose_plan(T, SUB, kElem, kTrimPlan<Tr>);
    const Access access = choose_access(same_lead, lead, T, SUB * plan.waves_per_row);
    if (access != Access::kRegular) plan = choose_plan(T, SUBG, kElem, kTrimPlan<Tr>);
    const int R = plan.rows_per_block;
    hipError_t err = hipSuccess;
#define ASCAN_BWD_PACKED(PW, AL, ACT)                                                                                  \
    launch_backward_packed<Tr, PW, AL, ACT>(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows, T, \
                                            at.grid, group, stream)
    // 16-bit rows of 512 bytes and more, vectorised flavour, plenty of them: groups of the wider workgroup
    if constexpr (Tr::kNarrow) {
        if (same_lead && T * kElem >= kPackedWideRowBytes) {
            const int group = packed_group(rows, T, kElem, SUBG * kPackedWavesWide, at.grid);
            if (group != 0 && rows / group >= kPackedWideMinGroups) {
                if (act == kGateSigmoid) {
                    err = ASCAN_BWD_PACKED(kPackedWavesWide, true, kGateSigmoid);
                } else {
                    err = ASCAN_BWD_PACKED(kPackedWavesWide, true, kGateIdentity);
                }
                return launch_status(err);
            }
        }
    }
    if (const int group = packed_group(rows, T, kElem, SUBG * kPackedWaves, same_lead ? at.grid : 1)) {
        if (act == kGateSigmoid) {
            if constexpr (kHasSigmoid<Tr>) {
                err = same_lead ? ASCAN_BWD_PACKED(kPackedWaves, true, kGateSigmoid)
                                : ASCAN_BWD_PACKED(kPackedWaves, false, kGateSigmoid);
            }
        } else {
            err = same_lead ? ASCAN_BWD_PACKED(kPackedWaves, true, kGateIdentity)
                            : ASCAN_BWD_PACKED(kPackedWaves, false, kGateIdentity);
        }
#undef ASCAN_BWD_PACKED
        return launch_status(err);
    }
    if (same_lead && ws.ptr != nullptr) {
        constexpr int64_t SUBS = (int64_t)SplitTuning<Tr>::UB * 64 * Tr::EPV;
        constexpr int64_t SUBSG = (int64_t)SplitTuning<Tr>::UBG * 64 * Tr::EPV;
        const bool regular = lead == 0 && T % (SUBS * kSplitWaves) == 0;
        const int64_t ntiles = host_tiles_per_row<Tr>(T, (regular ? SUBS : SUBSG) * kSplitWaves, regular, at);
        if (want_split(rows, ntiles) && workspace_fits(ws, rows, ntiles)) {
#define ASCAN_BWD_SPLIT(REG, ACT)                                                                              \
    launch_backward_split<Tr, REG, ACT>(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows, T, \
                                        at.grid, ntiles, ws, stream)
            if (act == kGateSigmoid) {
                if constexpr (kHasSigmoid<Tr>) {
                    err = regular ? ASCAN_BWD_SPLIT(true, kGateSigmoid) : ASCAN_BWD_SPLIT(false, kGateSigmoid);
                }
            } else {
                err = regular ? ASCAN_BWD_SPLIT(true, kGateIdentity) : ASCAN_BWD_SPLIT(false, kGateIdentity);
            }
#undef ASCAN_BWD_SPLIT
            return launch_status(err);
        }
    }
#define ASCAN_BWD_ARGS gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows, T, at.grid, R, stream
#define ASCAN_BWD(WV, AL, REG)                                                              \
    do {                                                                                    \
        if (act == kGateSigmoid) {                                                          \
            if constexpr (kHasSigmoid<Tr>)                                                  \
                err = launch_backward<Tr, WV, AL, REG, kGateSigmoid>(ASCAN_BWD_ARGS);       \
        } else {                                                                            \
            err = launch_backward<Tr, WV, AL, REG, kGateIdentity>(ASCAN_BWD_ARGS);          \
        }                                                                                   \
    } while (0)
#define ASCAN_BWD_W(AL, REG)                            \
    switch (plan.waves_per_row) {                       \
        case 1: ASCAN_BWD(1, AL, REG); break;           \
        case 2: ASCAN_BWD(2, AL, REG); break;           \
        case 4: ASCAN_BWD(4, AL, REG); break;           \
        case 8: ASCAN_BWD(8, AL, REG); break;           \
        default: ASCAN_BWD(16, AL, REG); break;         \
    }
    if (access == Access::kRegular) {
        ASCAN_BWD_W(true, true);
    } else if (access == Access::kVector) {
        ASCAN_BWD_W(true, false);
    } else {
        ASCAN_BWD_W(false, false);
    }
#undef ASCAN_BWD_W
#undef ASCAN_BWD
#undef ASCAN_BWD_ARGS
    return launch_status(err);
}

}  // namespace
}  // namespace ascan

// Defines ascan::NAME, the backward entry of one dtype, in the including file.
#define ASCAN_DEFINE_BACKWARD(NAME, TRAITS)                                                                  \
    int ascan::NAME(const ascan::BackwardCall& c) {                                                          \
        return ascan::backward_typed<ascan::TRAITS>(c.gates, c.states, c.grad_out, c.d_gates, c.d_tokens,   \
                                                    c.initial, c.d_initial, c.rows, c.seqlen, c.gate,       \
                                                    c.workspace, c.stream);                                 \
    }

#endif  // ASCAN_BACKWARD_DISPATCH_H_
