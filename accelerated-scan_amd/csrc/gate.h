// Gate non-linearity applied inside the kernels.

#ifndef ASCAN_GATE_H_
#define ASCAN_GATE_H_

#include "values.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Gate activation.  The kernels can read gate pre-activations ("logits") and
// apply the non-linearity in registers as the values are unpacked, which spares
// the caller a pass that materialises the gates and, in the backward pass, one
// that turns d_gates into the gradient of the logits.
//   kGateIdentity   : the stored values are the gates (the reference's operator);
//   kGateSigmoid    : gate = 1 / (1 + exp(-stored)), real dtypes only;
//   kGateSigmoidLerp: the same gate, and the token is (1 - gate) * stored value:
//                     x[t] = gate * x[t-1] + (1 - gate) * v[t], the gated
//                     interpolation of linear-RNN layers.  The tokens never
//                     exist in memory either;
//   kGateExp        : gate = exp(stored), real dtypes only: gates kept as
//                     logarithms (decay rates).  A 16-bit logarithm carries a
//                     gate close to 1 far more precisely than a 16-bit gate
//                     does (bf16 has no value between 0.996 and 1);
//   kGateExpNorm    : gate = exp(stored), and the token is sqrt(1 - gate^2) * stored
//                     value: x[t] = a x[t-1] + sqrt(1 - a^2) v[t], the update of
//                     RG-LRU / Hawk-style layers, whose input scale keeps the
//                     state's variance at that of the values.
// ---------------------------------------------------------------------------
constexpr int kGateIdentity = 0, kGateSigmoid = 1, kGateSigmoidLerp = 2, kGateExp = 3, kGateExpNorm = 4;

// Gates whose second input holds values v rather than tokens: the token is
// formed in registers from v and the gate, and the backward pass reads v again.
template <int ACT>
constexpr bool kGateTakesValues = ACT == kGateSigmoidLerp || ACT == kGateExpNorm;
inline bool gate_takes_values(int act) { return act == kGateSigmoidLerp || act == kGateExpNorm; }

template <int ACT>
constexpr bool kGateIsSigmoid = ACT == kGateSigmoid || ACT == kGateSigmoidLerp;

__device__ __forceinline__ float sigmoid(float v) {
    // v_exp_f32 computes 2^x; v_rcp_f32 is accurate to 1 ulp
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.4426950408889634f));
}

__device__ __forceinline__ float exp_gate(float v) {
    return __builtin_amdgcn_exp2f(v * 1.4426950408889634f);
}

// sigmoid(v) and 1 - sigmoid(v) = sigmoid(-v), each to about 2 ulp of its own
// magnitude: with t = exp(-|v|) the larger of the two is 1 / (1 + t) and the
// smaller t / (1 + t), so neither is formed as a difference from 1 and nothing
// overflows (v = +inf gives exactly (1, 0): the identity gate and a zero token).
__device__ __forceinline__ void sigmoid_pair(float v, float& gate, float& complement) {
    const float t = __builtin_amdgcn_exp2f(__builtin_fabsf(v) * -1.4426950408889634f);
    const float large = __builtin_amdgcn_rcpf(1.0f + t);
    const float small = t * large;
    const bool positive = v >= 0.0f;
    gate = positive ? large : small;
    complement = positive ? small : large;
}

// The same pair for kernels that keep it from pass 1 to pass 2 as one word per element: the
// smaller of the two, with the sign of v, is what comes back.  The larger one is formed
// as 1 - smaller here and in sigmoid_pair_from_kept, so both passes see the same bits
// (rounding to nearest puts it within 1 ulp of 1 / (1 + t)).
__device__ __forceinline__ float sigmoid_pair_kept(float v, float& gate, float& complement) {
    const float t = __builtin_amdgcn_exp2f(__builtin_fabsf(v) * -1.4426950408889634f);
    const float small = t * __builtin_amdgcn_rcpf(1.0f + t);
    const float large = 1.0f - small;
    const bool positive = v >= 0.0f;
    gate = positive ? large : small;
    complement = positive ? small : large;
    return positive ? small : -small;
}
__device__ __forceinline__ void sigmoid_pair_from_kept(float kept, float& gate, float& complement) {
    const float small = __builtin_fabsf(kept);
    const float large = 1.0f - small;
    const bool positive = f2i(kept) >= 0;  // the sign bit, so that a kept -0 is the negative side
    gate = positive ? large : small;
    complement = positive ? small : large;
}

// exp(v) and sqrt(1 - exp(2 v)) for v <= 0 (0 for v > 0).  1 - exp(w), w = 2 v, loses
// its leading digits to cancellation as w approaches 0, where the gates of long
// memories live; for w > -1/16 it is summed as -w (1 + w/2 + w^2/6 + w^3/24 + w^4/120)
// instead (truncation below 2e-9 relative; the difference 1 - a^2 is good to 1e-6 relative
// below that), so the scale keeps fp32 accuracy for every gate.  v = 0, the
// out-of-row fill, gives exactly (1, 0).
__device__ __forceinline__ void exp_norm_pair(float v, float& gate, float& scale) {
    gate = exp_gate(v);
    const float w = v + v;
    float series = __builtin_fmaf(w, 1.0f / 120.0f, 1.0f / 24.0f);
    series = __builtin_fmaf(series, w, 1.0f / 6.0f);
    series = __builtin_fmaf(series, w, 0.5f);
    series = __builtin_fmaf(series, w, 1.0f);
    const float direct = __builtin_fmaf(-gate, gate, 1.0f);
    const float m = w > -0.0625f ? -w * series : direct;
    scale = __builtin_amdgcn_sqrtf(__builtin_fmaxf(m, 0.0f));
}

template <int ACT, class V, int N>
__device__ __forceinline__ void activate(V (&g)[N]) {
    static_assert(!kGateTakesValues<ACT>, "gates with values go through activate_pair / activate_with_complement");
    if constexpr (ACT == kGateSigmoid) {
#pragma unroll
        for (int e = 0; e < N; ++e) g[e] = sigmoid(g[e]);
    } else if constexpr (ACT == kGateExp) {
#pragma unroll
        for (int e = 0; e < N; ++e) g[e] = exp_gate(g[e]);
    }
}
// Gates and tokens of a vector from the stored values: g holds gate
// pre-activations on entry and gates on exit; t holds the tokens, or for the
// interpolating gate the values v on entry and (1 - gate) * v on exit.
template <int ACT, class V, int N>
__device__ __forceinline__ void activate_pair(V (&g)[N], V (&t)[N]) {
    if constexpr (ACT == kGateSigmoidLerp) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            float gate, complement;
            sigmoid_pair(g[e], gate, complement);
            g[e] = gate;
            t[e] = complement * t[e];
        }
    } else if constexpr (ACT == kGateExpNorm) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            float gate, scale;
            exp_norm_pair(g[e], gate, scale);
            g[e] = gate;
            t[e] = scale * t[e];
        }
    } else {
        activate<ACT>(g);
    }
}
// Gates and the factor their values are weighted by -- 1 - gate for the interpolating
// gate, sqrt(1 - gate^2) for the normalised exponential one (the backward pass of both).
template <int ACT, class V, int N>
__device__ __forceinline__ void activate_with_complement(V (&g)[N], V (&c)[N]) {
    if constexpr (ACT == kGateSigmoidLerp) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            float gate, complement;
            sigmoid_pair(g[e], gate, complement);
            g[e] = gate;
            c[e] = complement;
        }
    } else if constexpr (ACT == kGateExpNorm) {
#pragma unroll
        for (int e = 0; e < N; ++e) {
            float gate, scale;
            exp_norm_pair(g[e], gate, scale);
            g[e] = gate;
            c[e] = scale;
        }
    } else {
        activate<ACT>(g);
    }
}
template <int ACT, class V>
__device__ __forceinline__ V activate1(V g) {
    if constexpr (ACT == kGateSigmoid) {
        return sigmoid(g);
    } else if constexpr (ACT == kGateSigmoidLerp) {
        float gate, complement;
        sigmoid_pair(g, gate, complement);
        return gate;
    } else if constexpr (ACT == kGateExp || ACT == kGateExpNorm) {
        return exp_gate(g);
    } else {
        return g;
    }
}
// Stored value whose activation is the identity gate 1 (for out-of-row positions).
template <int ACT, class V>
__device__ __forceinline__ V identity_gate() {
    if constexpr (kGateIsSigmoid<ACT>) {
        return __builtin_inff();
    } else if constexpr (ACT == kGateExp || ACT == kGateExpNorm) {
        return vzero<V>();
    } else {
        return vone<V>();
    }
}
// d gate / d stored, from the gate's value (and, where known, its complement).
template <int ACT, class V>
__device__ __forceinline__ V gate_slope(V gate) {
    if constexpr (ACT == kGateSigmoid) {
        return gate * (1.0f - gate);
    } else if constexpr (ACT == kGateExp) {
        return gate;
    } else {
        return vone<V>();
    }
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_GATE_H_
