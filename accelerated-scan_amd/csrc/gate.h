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
//   kGateIdentity: the stored values are the gates (the reference's operator);
//   kGateSigmoid : gate = 1 / (1 + exp(-stored)), real dtypes only.
// ---------------------------------------------------------------------------
constexpr int kGateIdentity = 0, kGateSigmoid = 1;

__device__ __forceinline__ float sigmoid(float v) {
    // v_exp_f32 computes 2^x; v_rcp_f32 is accurate to 1 ulp
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(v * -1.4426950408889634f));
}

template <int ACT, class V, int N>
__device__ __forceinline__ void activate(V (&g)[N]) {
    if constexpr (ACT == kGateSigmoid) {
#pragma unroll
        for (int e = 0; e < N; ++e) g[e] = sigmoid(g[e]);
    }
}
template <int ACT, class V>
__device__ __forceinline__ V activate1(V g) {
    if constexpr (ACT == kGateSigmoid) {
        return sigmoid(g);
    } else {
        return g;
    }
}
// Stored value whose activation is the identity gate 1 (for out-of-row positions).
template <int ACT, class V>
__device__ __forceinline__ V identity_gate() {
    if constexpr (ACT == kGateSigmoid) {
        return __builtin_inff();
    } else {
        return vone<V>();
    }
}
// d gate / d stored, from the gate's value.
template <int ACT, class V>
__device__ __forceinline__ V gate_slope(V gate) {
    if constexpr (ACT == kGateSigmoid) {
        return gate * (1.0f - gate);
    } else {
        return vone<V>();
    }
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_GATE_H_
