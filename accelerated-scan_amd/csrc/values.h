// Arithmetic values of the scan (float, complex) and the cross-lane steps of
// one wave64: DPP moves, the 6-step inclusive scan, lane reads.

#ifndef ASCAN_VALUES_H_
#define ASCAN_VALUES_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Value algebra: float for the real dtypes, cfloat for complex64.
// ---------------------------------------------------------------------------
struct cfloat {
    float re, im;
};

// An integer zero that the compiler cannot produce before `v` exists: added to the offset of a load, it
// keeps the load behind the arithmetic that yields `v`.
__device__ __forceinline__ int zero_after(float v) {
    int z = 0;
    asm volatile("" : "+v"(z) : "v"(v));
    return z;
}
__device__ __forceinline__ int zero_after(cfloat v) { return zero_after(v.re); }

__device__ __forceinline__ float vmul(float a, float b) { return a * b; }
__device__ __forceinline__ float vfma(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ float vconj(float a) { return a; }

__device__ __forceinline__ cfloat vmul(cfloat a, cfloat b) {
    cfloat r;
    r.re = __builtin_fmaf(a.re, b.re, -(a.im * b.im));
    r.im = __builtin_fmaf(a.re, b.im, a.im * b.re);
    return r;
}
// a * b + c
__device__ __forceinline__ cfloat vfma(cfloat a, cfloat b, cfloat c) {
    cfloat r;
    r.re = __builtin_fmaf(a.re, b.re, __builtin_fmaf(-a.im, b.im, c.re));
    r.im = __builtin_fmaf(a.re, b.im, __builtin_fmaf(a.im, b.re, c.im));
    return r;
}
__device__ __forceinline__ cfloat vconj(cfloat a) {
    cfloat r;
    r.re = a.re;
    r.im = -a.im;
    return r;
}

template <class V> __device__ __forceinline__ V vone();
template <class V> __device__ __forceinline__ V vzero();
template <> __device__ __forceinline__ float vone<float>() { return 1.0f; }
template <> __device__ __forceinline__ float vzero<float>() { return 0.0f; }
template <> __device__ __forceinline__ cfloat vone<cfloat>() { return cfloat{1.0f, 0.0f}; }
template <> __device__ __forceinline__ cfloat vzero<cfloat>() { return cfloat{0.0f, 0.0f}; }

__device__ __forceinline__ float vselect(bool c, float a, float b) { return c ? a : b; }
__device__ __forceinline__ cfloat vselect(bool c, cfloat a, cfloat b) {
    cfloat r;
    r.re = c ? a.re : b.re;
    r.im = c ? a.im : b.im;
    return r;
}

// ---------------------------------------------------------------------------
// Cross-lane primitives for one wave64.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int f2i(float x) { return __builtin_bit_cast(int, x); }
__device__ __forceinline__ float i2f(int x) { return __builtin_bit_cast(float, x); }

// DPP control words (GFX9 encoding).
constexpr int kRowShr1 = 0x111, kRowShr2 = 0x112, kRowShr4 = 0x114, kRowShr8 = 0x118;
constexpr int kWaveShl1 = 0x130, kWaveShr1 = 0x138;
constexpr int kRowBcast15 = 0x142, kRowBcast31 = 0x143;

// Lanes that have no source lane, or whose row is masked off, receive `old`.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_move(float old, float src) {
    return i2f(__builtin_amdgcn_update_dpp(f2i(old), f2i(src), CTRL, ROW_MASK, 0xF, false));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ cfloat dpp_move(cfloat old, cfloat src) {
    cfloat r;
    r.re = dpp_move<CTRL, ROW_MASK>(old.re, src.re);
    r.im = dpp_move<CTRL, ROW_MASK>(old.im, src.im);
    return r;
}

// One Kogge-Stone step of the pair scan: (Ap, Xp) o (A, X) = (Ap*A, Xp*A + X).
// The two halves of the scan operator, (A_l, X_l) o (A_r, X_r) =
// (A_l * A_r, A_r * X_l + X_r).  With RESET a gate of exactly zero discards
// what comes from the left even when that is not finite (0 * inf would be NaN):
// kernels that scan several rows as one, with a zero gate in front of each row,
// use it so that an overflowing row cannot reach into its neighbour.
__device__ __forceinline__ bool is_zero(float a) { return a == 0.0f; }
__device__ __forceinline__ bool is_zero(cfloat a) { return a.re == 0.0f && a.im == 0.0f; }

template <bool RESET, class V>
__device__ __forceinline__ V carry_in(V gate, V from_left, V local) {
    const V r = vfma(gate, from_left, local);
    if constexpr (RESET) {
        return vselect(is_zero(gate), local, r);
    } else {
        return r;
    }
}
template <bool RESET, class V>
__device__ __forceinline__ V gate_product(V left, V right) {
    const V r = vmul(left, right);
    if constexpr (RESET) {
        return vselect(is_zero(right), right, r);
    } else {
        return r;
    }
}

template <int CTRL, int ROW_MASK, bool RESET, class V>
__device__ __forceinline__ void scan_step(V& A, V& X) {
    const V Ap = dpp_move<CTRL, ROW_MASK>(vone<V>(), A);
    const V Xp = dpp_move<CTRL, ROW_MASK>(vzero<V>(), X);
    X = carry_in<RESET>(A, Xp, X);
    A = gate_product<RESET>(Ap, A);
}

// Inclusive scan of the 64 (A, X) pairs of a wave, ascending lane order.
template <bool RESET, class V>
__device__ __forceinline__ void wave_scan_inclusive(V& A, V& X) {
    scan_step<kRowShr1, 0xF, RESET>(A, X);
    scan_step<kRowShr2, 0xF, RESET>(A, X);
    scan_step<kRowShr4, 0xF, RESET>(A, X);
    scan_step<kRowShr8, 0xF, RESET>(A, X);
    scan_step<kRowBcast15, 0xA, RESET>(A, X);  // lane 15 of rows 0,2 -> rows 1,3
    scan_step<kRowBcast31, 0xC, RESET>(A, X);  // lane 31 -> rows 2,3
}

// Lane l receives v of lane l-1; lane 0 receives `edge`.
template <class V>
__device__ __forceinline__ V shift_up1(V v, V edge) {
    return dpp_move<kWaveShr1, 0xF>(edge, v);
}
// Lane l receives v of lane l+1; lane 63 receives `edge`.
template <class V>
__device__ __forceinline__ V shift_down1(V v, V edge) {
    return dpp_move<kWaveShl1, 0xF>(edge, v);
}

// v of lane `lane`, a wave-uniform index held in a scalar register.
__device__ __forceinline__ float read_lane_at(float v, int lane) {
    return i2f(__builtin_amdgcn_readlane(f2i(v), lane));
}
__device__ __forceinline__ cfloat read_lane_at(cfloat v, int lane) {
    cfloat r;
    r.re = read_lane_at(v.re, lane);
    r.im = read_lane_at(v.im, lane);
    return r;
}

template <int LANE>
__device__ __forceinline__ float read_lane(float v) {
    return i2f(__builtin_amdgcn_readlane(f2i(v), LANE));
}
template <int LANE>
__device__ __forceinline__ cfloat read_lane(cfloat v) {
    cfloat r;
    r.re = read_lane<LANE>(v.re);
    r.im = read_lane<LANE>(v.im);
    return r;
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_VALUES_H_
