// First-order linear recurrence (scan) kernels for gfx950 (MI355X) and the
// C ABI declared in include/ascan.h.
//
//   forward :  x[t] = gate[t] * x[t-1] + token[t]
//   backward:  g[t] = grad_out[t] + conj(gate[t+1]) * g[t+1]
//              d_tokens = g,  d_gates[t] = g[t] * conj(x[t-1])
//
// Behaviour follows the reference operator (accelerated_scan/warp.cuh:49-223
// for the real dtypes, accelerated_scan/complex.py:20-154 for complex64); the
// decomposition below is specific to CDNA wave64 hardware:
//
//   * A row is cut into tiles; inside a tile every wave owns a contiguous
//     sub-tile of U*64 16-byte vectors.  Lane l of the wave loads vector
//     j*64+l of the sub-tile (j = 0..U-1), so each load instruction of the
//     wave covers one contiguous KiB.  Loads and stores carry the nontemporal
//     hint: nothing is read twice.
//   * Each lane folds its vector into one (A, X) pair, A = product of gates,
//     X = local scan end value.  The 64 pairs are scanned with 6 DPP steps
//     (row_shr 1,2,4,8, row_bcast 15, row_bcast 31): no LDS, no barrier.
//   * The carry entering a block is a wave-uniform value; it is chained over
//     the U blocks and over the tiles of the row in registers.  A row gets up
//     to 16 waves (one per 4 KiB of row); their sub-tile totals go through a
//     double-buffered LDS slot array, one barrier per tile.
//   * Every output element is then recomputed by the plain recurrence from the
//     state entering its lane, so the per-element arithmetic is the sequential
//     one and only the lane-entry state depends on the tree order.
//   * Reverse-time kernels mirror the lane mapping (lane l takes vector
//     63-l, elements in descending order) so the same ascending-lane scan
//     applies.  The backward pass gets gate[t+1] and x[t-1] from the vectors
//     it already holds plus one-lane DPP shifts; only the two elements just
//     outside a wave's sub-tile are loaded separately.
//   * Calls with few rows and long sequences run the same kernels in a second
//     mode in which the tiles of a row are spread over many workgroups that
//     pass the running state through a table in global memory.
//
// All arithmetic is fp32 with fused multiply-add.

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdlib.h>

#include <atomic>
#include <type_traits>

#include "ascan.h"

namespace {

// ---------------------------------------------------------------------------
// Value algebra: float for the real dtypes, cfloat for complex64.
// ---------------------------------------------------------------------------
struct cfloat {
    float re, im;
};

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
template <int CTRL, int ROW_MASK, class V>
__device__ __forceinline__ void scan_step(V& A, V& X) {
    const V Ap = dpp_move<CTRL, ROW_MASK>(vone<V>(), A);
    const V Xp = dpp_move<CTRL, ROW_MASK>(vzero<V>(), X);
    X = vfma(Xp, A, X);
    A = vmul(Ap, A);
}

// Inclusive scan of the 64 (A, X) pairs of a wave, ascending lane order.
template <class V>
__device__ __forceinline__ void wave_scan_inclusive(V& A, V& X) {
    scan_step<kRowShr1, 0xF>(A, X);
    scan_step<kRowShr2, 0xF>(A, X);
    scan_step<kRowShr4, 0xF>(A, X);
    scan_step<kRowShr8, 0xF>(A, X);
    scan_step<kRowBcast15, 0xA>(A, X);  // lane 15 of rows 0,2 -> rows 1,3
    scan_step<kRowBcast31, 0xC>(A, X);  // lane 31 -> rows 2,3
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

// ---------------------------------------------------------------------------
// Storage traits: S = element type in memory, V = arithmetic type,
// EPV = elements per 16-byte vector.
// ---------------------------------------------------------------------------
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));  // one 16-byte vector
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef float floatx2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef _Float16 halfx2_t __attribute__((ext_vector_type(2)));

struct TraitsF32 {
    using S = float;
    using TokS = S;  // tokens and d_tokens are stored like everything else
    using V = float;
    static constexpr int EPV = 4;
    static constexpr bool kRealTokens = false;
    static constexpr bool kNarrow = false;  // unpacked form is no larger than the raw vector
    static __device__ __forceinline__ void unpack(const u32x4_t& r, V (&d)[EPV]) {
        d[0] = i2f(r.x);
        d[1] = i2f(r.y);
        d[2] = i2f(r.z);
        d[3] = i2f(r.w);
    }
    static __device__ __forceinline__ u32x4_t pack(const V (&s)[EPV]) {
        u32x4_t r;
        r.x = f2i(s[0]);
        r.y = f2i(s[1]);
        r.z = f2i(s[2]);
        r.w = f2i(s[3]);
        return r;
    }
    static __device__ __forceinline__ V load1(const S* p) { return *p; }
    static __device__ __forceinline__ void store1(S* p, V v) { *p = v; }
};

struct TraitsBF16 {
    using S = uint16_t;
    using TokS = S;
    using V = float;
    static constexpr int EPV = 8;
    static constexpr bool kRealTokens = false;
    static constexpr bool kNarrow = true;
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        floatx2_t f;
        f.x = lo;
        f.y = hi;
        const bf16x2_t h = __builtin_convertvector(f, bf16x2_t);  // round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ void unpack(const u32x4_t& r, V (&d)[EPV]) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            d[2 * i] = i2f((int)(w[i] << 16));
            d[2 * i + 1] = i2f((int)(w[i] & 0xffff0000u));
        }
    }
    static __device__ __forceinline__ u32x4_t pack(const V (&s)[EPV]) {
        u32x4_t r;
        r.x = pack2(s[0], s[1]);
        r.y = pack2(s[2], s[3]);
        r.z = pack2(s[4], s[5]);
        r.w = pack2(s[6], s[7]);
        return r;
    }
    static __device__ __forceinline__ V load1(const S* p) { return i2f((int)((uint32_t)(*p) << 16)); }
    static __device__ __forceinline__ void store1(S* p, V v) { *p = (uint16_t)(pack2(v, 0.0f) & 0xffffu); }
};

struct TraitsF16 {
    using S = uint16_t;
    using TokS = S;
    using V = float;
    static constexpr int EPV = 8;
    static constexpr bool kRealTokens = false;
    static constexpr bool kNarrow = true;
    static __device__ __forceinline__ uint32_t pack2(float lo, float hi) {
        floatx2_t f;
        f.x = lo;
        f.y = hi;
        const halfx2_t h = __builtin_convertvector(f, halfx2_t);  // round to nearest even
        return __builtin_bit_cast(uint32_t, h);
    }
    static __device__ __forceinline__ void unpack(const u32x4_t& r, V (&d)[EPV]) {
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const halfx2_t h = __builtin_bit_cast(halfx2_t, w[i]);
            const floatx2_t f = __builtin_convertvector(h, floatx2_t);
            d[2 * i] = f.x;
            d[2 * i + 1] = f.y;
        }
    }
    static __device__ __forceinline__ u32x4_t pack(const V (&s)[EPV]) {
        u32x4_t r;
        r.x = pack2(s[0], s[1]);
        r.y = pack2(s[2], s[3]);
        r.z = pack2(s[4], s[5]);
        r.w = pack2(s[6], s[7]);
        return r;
    }
    static __device__ __forceinline__ V load1(const S* p) {
        return (float)__builtin_bit_cast(_Float16, *p);
    }
    static __device__ __forceinline__ void store1(S* p, V v) {
        *p = __builtin_bit_cast(uint16_t, (_Float16)v);
    }
};

struct TraitsC64 {
    using S = cfloat;  // 8 bytes, interleaved (re, im)
    using TokS = S;
    using V = cfloat;
    static constexpr int EPV = 2;
    static constexpr bool kRealTokens = false;
    static constexpr bool kNarrow = false;
    static __device__ __forceinline__ void unpack(const u32x4_t& r, V (&d)[EPV]) {
        d[0].re = i2f(r.x);
        d[0].im = i2f(r.y);
        d[1].re = i2f(r.z);
        d[1].im = i2f(r.w);
    }
    static __device__ __forceinline__ u32x4_t pack(const V (&s)[EPV]) {
        u32x4_t r;
        r.x = f2i(s[0].re);
        r.y = f2i(s[0].im);
        r.z = f2i(s[1].re);
        r.w = f2i(s[1].im);
        return r;
    }
    static __device__ __forceinline__ V load1(const S* p) {
        const float2 v = *reinterpret_cast<const float2*>(p);
        cfloat r;
        r.re = v.x;
        r.im = v.y;
        return r;
    }
    static __device__ __forceinline__ void store1(S* p, V v) {
        float2 o;
        o.x = v.re;
        o.y = v.im;
        *reinterpret_cast<float2*>(p) = o;
    }
};

// complex64 gates / states / gradients with real (fp32) tokens: the tokens are
// read as (token, 0) and the token gradient keeps its real part, without a
// complex copy of the tokens ever existing in memory
// (accelerated_scan/complex.py:162,168-169,217-218 promote and slice instead).
struct TraitsC64RealTokens : TraitsC64 {
    using TokS = float;
    static constexpr bool kRealTokens = true;
    // two fp32 tokens (8 bytes) <-> the raw form of two complex values
    static __device__ __forceinline__ u32x4_t tok_widen(u32x2_t r) {
        u32x4_t o;
        o.x = r.x;
        o.y = 0u;
        o.z = r.y;
        o.w = 0u;
        return o;
    }
    static __device__ __forceinline__ u32x2_t tok_narrow(const V (&s)[EPV]) {
        u32x2_t o;
        o.x = f2i(s[0].re);
        o.y = f2i(s[1].re);
        return o;
    }
    static __device__ __forceinline__ V tok_load1(const TokS* p) {
        cfloat r;
        r.re = *p;
        r.im = 0.0f;
        return r;
    }
    static __device__ __forceinline__ void tok_store1(TokS* p, V v) { *p = v.re; }
};

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

// ---------------------------------------------------------------------------
// Vector access.  A row is addressed in "virtual" positions: position 0 is an
// aligned boundary at or just below the row's first element -- a 128-byte one
// when all tensors of the call sit alike on that grid, so that the 1 KiB a wave
// moves per instruction is eight whole cache lines wherever the row starts
// (rows on the 16-byte grid only measured 10 % slower), else a 16-byte one --
// and the row's elements occupy [lo, hi) with 0 <= lo < G, G being the number
// of elements between two such boundaries.  Inside the tile loop everything
// is expressed relative to the wave's sub-tile: `sub` points at the first
// element of the sub-tile (wave-uniform, 64-bit), `off` is the lane's 32-bit
// element offset inside it, and a Window holds the row's valid range relative
// to the sub-tile.  Only `off` is per-lane state.
//   ALIGNED: sub + off is 16-byte aligned, so vectors move as one dwordx4.  A
//            vector that straddles a row end (at most two per row) is read
//            whole and masked, and stored element by element so a neighbouring
//            row's bytes are never written.  The !ALIGNED kernels move
//            everything element by element.
//   FULL   : the whole sub-tile is known to lie inside the row.
// ---------------------------------------------------------------------------
struct Window {
    int lo, hi;  // valid element offsets: lo <= off < hi (clamped to +-2^30)
};

__device__ __forceinline__ Window make_window(int64_t lo, int64_t hi, int64_t sub_base) {
    constexpr int64_t kClamp = 1 << 30;
    int64_t l = lo - sub_base, h = hi - sub_base;
    l = l < -kClamp ? -kClamp : (l > kClamp ? kClamp : l);
    h = h < -kClamp ? -kClamp : (h > kClamp ? kClamp : h);
    Window win;
    win.lo = (int)l;
    win.hi = (int)h;
    return win;
}

__device__ __forceinline__ bool in_window(Window win, int off) { return off >= win.lo && off < win.hi; }

// Returns the vector as raw bits with out-of-row elements replaced by `fill`.
// The caller guarantees that the sub-tile overlaps the row unless FULL.
template <class Tr, bool ALIGNED, bool FULL>
__device__ __forceinline__ u32x4_t load_raw(const typename Tr::S* __restrict__ sub, int off, Window win,
                                            typename Tr::V fill) {
    constexpr int EPV = Tr::EPV;
    if constexpr (ALIGNED) {
        // A vector that straddles a row end is still read whole: an aligned
        // 16-byte read that overlaps the row cannot leave the row's memory
        // page, and the bytes of the neighbouring row are discarded below.  A
        // vector entirely outside the row re-reads a vector of this sub-tile
        // that does overlap it, so the load stays unconditional.
        int o = off;
        if (!FULL) {
            const int safe = win.lo > 0 ? (win.lo / EPV) * EPV : 0;
            o = (off + EPV > win.lo && off < win.hi) ? off : safe;
        }
        u32x4_t raw = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(sub + o));
        if (!FULL) {
            typename Tr::V v[EPV];
            Tr::unpack(raw, v);
#pragma unroll
            for (int e = 0; e < EPV; ++e) v[e] = vselect(in_window(win, off + e), v[e], fill);
            raw = Tr::pack(v);  // exact: every storage value survives the round trip
        }
        return raw;
    } else {
        typename Tr::V v[EPV];
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            if (FULL || in_window(win, off + e)) {
                v[e] = Tr::load1(sub + off + e);
            } else {
                v[e] = fill;
            }
        }
        return Tr::pack(v);
    }
}

// The vector every lane holds when the sub-tile lies entirely outside the row.
template <class Tr>
__device__ __forceinline__ u32x4_t fill_raw(typename Tr::V fill) {
    typename Tr::V v[Tr::EPV];
#pragma unroll
    for (int e = 0; e < Tr::EPV; ++e) v[e] = fill;
    return Tr::pack(v);
}

// Makes the compiler forget what it knows about `raw`, so that values unpacked
// from it before this point are not kept alive for re-use after it.  For the
// 16-bit formats the raw vector is half the registers of its unpacked form.
__device__ __forceinline__ void forget_unpacked(u32x4_t& raw) {
    unsigned x = raw.x, y = raw.y, z = raw.z, w = raw.w;
    asm volatile("" : "+v"(x), "+v"(y), "+v"(z), "+v"(w));
    raw.x = x;
    raw.y = y;
    raw.z = z;
    raw.w = w;
}

template <class Tr, bool ALIGNED, bool FULL>
__device__ __forceinline__ void store_vec(typename Tr::S* __restrict__ sub, int off, Window win,
                                          const typename Tr::V (&src)[Tr::EPV]) {
    constexpr int EPV = Tr::EPV;
    if (ALIGNED && (FULL || (off >= win.lo && off + EPV <= win.hi))) {
        __builtin_nontemporal_store(Tr::pack(src), reinterpret_cast<u32x4_t*>(sub + off));
    } else {
#pragma unroll
        for (int e = 0; e < EPV; ++e) {
            if (FULL || in_window(win, off + e)) Tr::store1(sub + off + e, src[e]);
        }
    }
}

// Token-side access: identical to load_raw / store_vec unless the tokens are
// real while the scan is complex, in which case a "vector" of EPV tokens is 8
// bytes of fp32.
template <class Tr, bool ALIGNED, bool FULL>
__device__ __forceinline__ u32x4_t load_tok_raw(const typename Tr::TokS* __restrict__ sub, int off, Window win,
                                                typename Tr::V fill) {
    if constexpr (!Tr::kRealTokens) {
        return load_raw<Tr, ALIGNED, FULL>(sub, off, win, fill);
    } else {
        constexpr int EPV = Tr::EPV;
        if constexpr (ALIGNED) {
            int o = off;
            if (!FULL) {
                const int safe = win.lo > 0 ? (win.lo / EPV) * EPV : 0;
                o = (off + EPV > win.lo && off < win.hi) ? off : safe;
            }
            u32x4_t raw = Tr::tok_widen(__builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(sub + o)));
            if (!FULL) {
                typename Tr::V v[EPV];
                Tr::unpack(raw, v);
#pragma unroll
                for (int e = 0; e < EPV; ++e) v[e] = vselect(in_window(win, off + e), v[e], fill);
                raw = Tr::pack(v);
            }
            return raw;
        } else {
            typename Tr::V v[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                if (FULL || in_window(win, off + e)) {
                    v[e] = Tr::tok_load1(sub + off + e);
                } else {
                    v[e] = fill;
                }
            }
            return Tr::pack(v);
        }
    }
}

template <class Tr, bool ALIGNED, bool FULL>
__device__ __forceinline__ void store_tok_vec(typename Tr::TokS* __restrict__ sub, int off, Window win,
                                              const typename Tr::V (&src)[Tr::EPV]) {
    if constexpr (!Tr::kRealTokens) {
        store_vec<Tr, ALIGNED, FULL>(sub, off, win, src);
    } else {
        constexpr int EPV = Tr::EPV;
        if (ALIGNED && (FULL || (off >= win.lo && off + EPV <= win.hi))) {
            __builtin_nontemporal_store(Tr::tok_narrow(src), reinterpret_cast<u32x2_t*>(sub + off));
        } else {
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                if (FULL || in_window(win, off + e)) Tr::tok_store1(sub + off + e, src[e]);
            }
        }
    }
}

// Number of tiles every wave of the grid iterates over (the barrier count must
// be the same for all waves of a workgroup).  `head` is the largest misalignment
// of a row start, in elements, over all rows.
__device__ __forceinline__ int64_t tiles_per_row(int64_t T, int64_t tile, int head) {
    return (T + head + tile - 1) / tile;
}

// Misalignment of the row start in elements (0 <= result < G, G a power of
// two).  All tensors of a call share it: the host checks that their base
// addresses are congruent on that grid.
template <class Tr>
__device__ __forceinline__ int row_lead(const typename Tr::S* row_start, int G) {
    return (int)((reinterpret_cast<uintptr_t>(row_start) / sizeof(typename Tr::S)) & (uintptr_t)(G - 1));
}

// Element index (inside the sub-tile) of the vector that lane `lane` owns in
// scan-order block j.  Reverse-time kernels mirror the mapping.
template <int U, int EPV, bool REV>
__device__ __forceinline__ int vec_offset(int j, int lane) {
    const int q = j * 64 + lane;
    return (REV ? (U * 64 - 1 - q) : q) * EPV;
}

// A workgroup has at most 16 waves: R rows x W waves per row.
constexpr int kMaxWavesPerBlock = 16;
constexpr int kSlotsPerBuffer = 2 * kMaxWavesPerBlock;  // one (A, X) pair per wave

// Maps the wave to its row and its position in the row.  Returns false for a
// wave whose row is past the end: it only keeps the workgroup's barriers
// company (one per tile) and touches no memory.
template <int W>
__device__ __forceinline__ bool locate_wave(int64_t rows, int64_t ntiles, int64_t& row, int& w, int& slot_base) {
    const int wv = threadIdx.x >> 6;
    const int rows_per_block = (int)(blockDim.x >> 6) / W;
    const int rib = wv / W;  // row inside the block
    w = wv - rib * W;
    slot_base = 2 * rib * W;
    row = (int64_t)blockIdx.x * rows_per_block + rib;
    if (row < rows) return true;
    if constexpr (W > 1) {
        for (int64_t k = 0; k < ntiles; ++k) __syncthreads();
    }
    return false;
}

// Carry bookkeeping shared by the forward and the backward kernel.
//
// Input : totA/totX[j]   inclusive total of block j of this wave (wave-uniform)
//         carry          state entering the tile (wave-uniform, same in all waves)
// Output: c              state entering block 0 of this wave
//         carry          state entering the next tile
// With W > 1 the W waves of a row exchange their sub-tile totals through
// `slots`, the row's W entries of one of two buffers selected by `parity`.
template <class V, int W, int U>
__device__ __forceinline__ void exchange_carries(const V (&totA)[U], const V (&totX)[U], V& carry, V& c,
                                                 V* slots, int parity, int w, int lane) {
    if constexpr (W == 1) {
        c = carry;
        V n = carry;
#pragma unroll
        for (int j = 0; j < U; ++j) n = vfma(totA[j], n, totX[j]);
        carry = n;
    } else {
        V TA = totA[0], TX = totX[0];
#pragma unroll
        for (int j = 1; j < U; ++j) {
            TX = vfma(TX, totA[j], totX[j]);
            TA = vmul(TA, totA[j]);
        }
        V* buf = slots + parity * kSlotsPerBuffer;
        if (lane == 0) {
            buf[2 * w] = TA;
            buf[2 * w + 1] = TX;
        }
        __syncthreads();
        V run = carry;
        V mine = carry;
#pragma unroll
        for (int i = 0; i < W; ++i) {
            const V Ai = buf[2 * i];
            const V Xi = buf[2 * i + 1];
            mine = vselect(i == w, run, mine);
            run = vfma(Ai, run, Xi);
        }
        c = mine;
        carry = run;
    }
}

// ---------------------------------------------------------------------------
// Split rows: several workgroups per row, for calls with too few rows to
// occupy the machine.  Every workgroup takes ONE tile of one row; the state
// entering the tile comes from the workgroups of the earlier tiles through a
// small table in global memory (single pass, "decoupled look-back"):
//   * a workgroup publishes its tile's aggregate (A, X) as soon as it has it;
//   * it then walks back over the earlier tiles of its row, folding aggregates
//     until it meets a tile whose inclusive state P is already published;
//   * it publishes its own inclusive state and finishes the tile.
// Tiles are handed out by ticket: every row has a counter, and a workgroup
// takes the next tile of a row with one fetch-add on it (moving on to the next
// row when a row has no tiles left).  A tile is therefore only ever waited for
// by workgroups that started after its owner did: progress never depends on a
// workgroup that has not been dispatched yet, whatever else is running on the
// GPU, and the launch size (what an idle GPU holds at once) is a matter of
// speed only.  One counter per row keeps the fetch-adds of different rows
// apart (measured: ~11 ns each on one address, concurrent across addresses).
// Each wait is nevertheless bounded by a limit set by the host; a wait that
// runs out poisons the result with NaN and is counted in the header.  Waiting
// time is summed from clock differences capped at 10 us each, so a stretch
// during which the whole kernel was not running does not count.
// ---------------------------------------------------------------------------
struct SplitHeader {
    unsigned long long reserved0;
    unsigned long long wait_limit;  // longest single wait, in s_memrealtime ticks (100 MHz)
    unsigned int timeouts;          // waits that ran out
    unsigned int reserved[11];
};
static_assert(sizeof(SplitHeader) == 64, "header is 64 bytes");

// One ticket counter per row, each on a cache line of its own.
struct alignas(64) SplitTicket {
    unsigned long long next;  // scan-order index of the next tile to hand out
    unsigned long long pad[7];
};
static_assert(sizeof(SplitTicket) == 64, "ticket line is 64 bytes");

constexpr unsigned long long kWaitStepCap = 1000;  // 10 us in 100 MHz ticks

// One record per (row, tile).  Every field is a 64-bit word holding an fp32
// payload in its low half and a tag in its high half (0 = not written yet,
// 1 = valid), written and read with single relaxed device-scope atomics: the
// payload arrives together with its tag, so no fence (on this hardware a
// write-back or invalidate of a whole L2) is needed on either side.
struct alignas(64) SplitRecord {
    unsigned long long a[2];  // aggregate gate product of the tile (re, im)
    unsigned long long x[2];  // aggregate state of the tile from a zero start (re, im)
    unsigned long long p[2];  // inclusive state at the end of the tile (re, im)
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
    if (i < nwords) words[i] = 0u;
    if (i == 0) {
        // the limit occupies words 2 and 3 of the header
        words[2] = (uint32_t)wait_limit;
        words[3] = (uint32_t)(wait_limit >> 32);
    }
}

// Layout of the table: header, one ticket line per row, one record per (row, tile).
__device__ __forceinline__ SplitTicket* split_tickets(SplitHeader* header) {
    return reinterpret_cast<SplitTicket*>(header + 1);
}
__device__ __forceinline__ SplitRecord* split_records(SplitHeader* header, int64_t rows) {
    return reinterpret_cast<SplitRecord*>(split_tickets(header) + rows);
}

// A workgroup's place in the hand-out of tiles: the row it is taking tiles from
// and the ticket it has already drawn for its next tile (drawn while the
// current tile's loads are in flight, so that the fetch-add's latency is off
// the critical path).  Meaningful in wave 0 only.
struct SplitWalk {
    int64_t row;
    unsigned long long drawn;  // valid when has_drawn
    bool has_drawn;
};

__device__ __forceinline__ unsigned long long draw_ticket(SplitTicket* ticket, int lane) {
    unsigned long long t = 0;
    if (lane == 0) t = __hip_atomic_fetch_add(&ticket->next, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return t;  // lane 0 holds the ticket
}
__device__ __forceinline__ unsigned long long from_lane0(unsigned long long v) {
    return ((unsigned long long)(unsigned)__builtin_amdgcn_readfirstlane((int)(v >> 32)) << 32) |
           (unsigned)__builtin_amdgcn_readfirstlane((int)v);
}

// Hands the workgroup its next tile: the next tile of the row it is on if that
// row has one left, else of the next row (cyclically) that does.  Returns false
// when no row has tiles left.  All threads of the workgroup call it together
// and get the same answer; `mailbox` is two words of LDS.
__device__ __forceinline__ bool take_split_tile(SplitHeader* header, int64_t rows, int64_t ntiles, SplitWalk& walk,
                                                int64_t& row, int64_t& k, long long* mailbox) {
    if (threadIdx.x < 64) {  // wave 0
        const int lane = threadIdx.x;
        SplitTicket* tickets = split_tickets(header);
        long long got_row = -1, got_k = -1;
        for (;;) {
            unsigned long long ticket;
            if (walk.has_drawn) {
                ticket = from_lane0(walk.drawn);
                walk.has_drawn = false;
            } else {
                // first row at or after walk.row, cyclically, that still has tiles: 64 rows per look
                long long found = -1;
                for (int64_t base = 0; base < rows && found < 0; base += 64) {
                    const int64_t idx = base + lane;
                    bool has = false;
                    if (idx < rows) {
                        const int64_t r = walk.row + idx < rows ? walk.row + idx : walk.row + idx - rows;
                        has = __hip_atomic_load(&tickets[r].next, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) <
                              (unsigned long long)ntiles;
                    }
                    const unsigned long long mask = __ballot(has);
                    if (mask) found = base + (long long)__builtin_ctzll(mask);
                }
                if (found < 0) break;  // nothing left anywhere
                walk.row = walk.row + found < rows ? walk.row + found : walk.row + found - rows;
                ticket = from_lane0(draw_ticket(&tickets[walk.row], lane));
            }
            if (ticket < (unsigned long long)ntiles) {
                got_row = walk.row;
                got_k = (long long)ticket;
                if (ticket + 1 < (unsigned long long)ntiles) {  // draw the next one now; it is read at the next call
                    walk.drawn = draw_ticket(&tickets[walk.row], lane);
                    walk.has_drawn = true;
                }
                break;
            }
            // the row ran out (another workgroup took its last tile): look again
        }
        if (lane == 0) {
            mailbox[0] = got_row;
            mailbox[1] = got_k;
        }
    }
    __syncthreads();
    const long long got_row = mailbox[0];
    const long long got_k = mailbox[1];
    __syncthreads();  // the mailbox may be rewritten by the next call
    if (got_row < 0) return false;
    row = got_row;
    k = got_k;
    return true;
}

__device__ __forceinline__ float read_lane_at(float v, int lane) {
    return i2f(__builtin_amdgcn_readlane(f2i(v), lane));
}
__device__ __forceinline__ cfloat read_lane_at(cfloat v, int lane) {
    cfloat r;
    r.re = read_lane_at(v.re, lane);
    r.im = read_lane_at(v.im, lane);
    return r;
}

// State entering scan-order tile k of a row, for wave 0 of the workgroup that
// owns the tile.  `mine` is that row's first record; records of successive
// tiles are `stride` apart.  (tileA, tileX) is this tile's aggregate and
// `row_start` the state entering tile 0.
//
// The walk back is done 64 tiles at a time: lane i looks at tile k-1-i, all
// lanes wait for their record in parallel (one memory round trip instead of one
// per tile), then the records from the nearest inclusive state forward are
// folded with lane reads.
template <class V>
__device__ __forceinline__ V split_look_back(SplitHeader* header, SplitRecord* mine, int64_t stride, int64_t k,
                                             V tileA, V tileX, V row_start, int lane) {
    SplitRecord* rec = mine + k * stride;
    V carry_in = row_start;  // the state entering tile 0
    if (k > 0) {
        if (lane == 0) {
            publish(rec->a, tileA);
            publish(rec->x, tileX);
        }
        const unsigned long long limit = header->wait_limit;
        V accA = vone<V>(), accX = vzero<V>();  // aggregate of the tiles nearer than the current window
        bool done = false;
        for (int64_t base = k - 1; base >= 0 && !done; base -= 64) {
            const int64_t q = base - lane;
            const bool active = q >= 0;
            // 0 nothing seen, 1 aggregate in (A, X), 2 inclusive state in X
            int seen = 0;
            V A = vone<V>(), X = vzero<V>();
            if (active) {
                SplitRecord* prev = mine + q * stride;
                unsigned long long waited = 0, last = __builtin_amdgcn_s_memrealtime();
                for (;;) {
                    V P, Aq, Xq;
                    if (peek(prev->p, P)) {
                        X = P;
                        seen = 2;
                        break;
                    }
                    const bool has_a = peek(prev->a, Aq);
                    const bool has_x = peek(prev->x, Xq);
                    if (has_a && has_x) {
                        A = Aq;
                        X = Xq;
                        seen = 1;
                        break;
                    }
                    const unsigned long long now = __builtin_amdgcn_s_memrealtime();
                    waited += now - last < kWaitStepCap ? now - last : kWaitStepCap;
                    last = now;
                    if (waited > limit) break;
                    __builtin_amdgcn_s_sleep(1);
                }
            }
            const int n_active = base + 1 < 64 ? (int)(base + 1) : 64;
            const unsigned long long inclusive = __ballot(active && seen == 2);
            const unsigned long long late = __ballot(active && seen == 0);
            // lanes [0, first) hold aggregates to fold; lane `first`, if active, holds an inclusive state
            const int first = inclusive ? (int)__builtin_ctzll(inclusive) : n_active;
            const unsigned long long needed = first >= 63 ? ~0ull : ((2ull << first) - 1ull);
            if (late & needed) {
                // a wait ran out: give up on this tile, visibly
                if (lane == 0) atomicAdd(&header->timeouts, 1u);
                carry_in = poison(carry_in);
                done = true;
            } else {
                V wA = vone<V>(), wX = vzero<V>();  // aggregate of tiles k-1-(first-1) .. k-1 of this window
                for (int i = first - 1; i >= 0; --i) {
                    const V Ai = read_lane_at(A, i);
                    const V Xi = read_lane_at(X, i);
                    wX = vfma(wX, Ai, Xi);
                    wA = vmul(wA, Ai);
                }
                // (w) o (acc): the window's tiles come before the nearer ones
                accX = vfma(wX, accA, accX);
                accA = vmul(wA, accA);
                if (first < n_active) {
                    const V P = read_lane_at(X, first);
                    carry_in = vfma(accA, P, accX);
                    done = true;
                }
            }
        }
        // tile 0 always publishes an inclusive state, so the walk ends there at the latest
    }
    if (lane == 0) publish(rec->p, vfma(tileA, carry_in, tileX));
    return carry_in;
}

// exchange_carries for a workgroup that owns a single tile of a split row: the
// tile carry comes from split_look_back instead of the previous loop iteration.
template <class V, int W, int U>
__device__ __forceinline__ void exchange_carries_split(const V (&totA)[U], const V (&totX)[U], V& c, V* slots,
                                                       int w, int lane, SplitHeader* header, SplitRecord* mine,
                                                       int64_t stride, int64_t k, V row_start) {
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
#pragma unroll
    for (int i = 0; i < W; ++i) {
        const V Ai = slots[2 * i];
        const V Xi = slots[2 * i + 1];
        mineA = vselect(i == w, runA, mineA);
        mineX = vselect(i == w, runX, mineX);
        runX = vfma(runX, Ai, Xi);
        runA = vmul(runA, Ai);
    }
    V* carry_slot = slots + kSlotsPerBuffer;
    if (w == 0) {  // wave-uniform
        const V carry_in = split_look_back(header, mine, stride, k, runA, runX, row_start, lane);
        if (lane == 0) *carry_slot = carry_in;
    }
    __syncthreads();
    c = vfma(mineA, *carry_slot, mineX);
}

// ---------------------------------------------------------------------------
// Packed rows: short rows, many of them.  One workgroup per row would leave
// most lanes idle (a row of 16 elements occupies 4 lanes of one wave), so a
// workgroup scans a group of consecutive rows -- one contiguous stretch of
// memory -- as a single long row with a "cut" in front of every row: at a row's
// first element the gate is replaced by 0, which annihilates whatever the scan
// carries in from the row before, and gate * x[-1] is added to the token.  All
// of the tiling, masking and carry code is shared with the one-row-per-
// workgroup mode; the cuts are applied to the unpacked vectors.
//   rel  position of an element relative to the first element of the group;
//   the element is the first of its row when rel % T == 0, the last when
//   rel % T == T - 1, and belongs to row rel / T of the group.
// The initial states of the rows a wave's sub-tile touches are staged in LDS by
// one coalesced read, so the cuts need no per-lane global loads.
// ---------------------------------------------------------------------------
template <class Tr>
struct Cuts {
    int T;          // row length
    float inv_T;    // 1 / T
    int len;        // elements in the group
    int first_row;  // of the rows staged in `stage`, relative to the group
    const typename Tr::S* stage;  // their initial states (LDS), or null
};

// Row and position-in-row of element `rel` (exact for the magnitudes that occur:
// |rel| < 2^21, T < 2^21).
__device__ __forceinline__ void split_position(int rel, int T, float inv_T, int& row, int& pos) {
    row = (int)__builtin_floorf(((float)rel + 0.5f) * inv_T);
    pos = rel - row * T;
}

// Forward / reverse scan: at the element that starts the recurrence of its row
// (first in time order), token += gate * x_start and gate = 0.
template <class Tr, bool REV>
__device__ __forceinline__ void cut_rows(typename Tr::V (&g)[Tr::EPV], typename Tr::V (&t)[Tr::EPV], int rel0,
                                         const Cuts<Tr>& cuts) {
    using V = typename Tr::V;
    int row, pos;
    split_position(rel0, cuts.T, cuts.inv_T, row, pos);
#pragma unroll
    for (int e = 0; e < Tr::EPV; ++e) {
        const bool valid = (unsigned)(rel0 + e) < (unsigned)cuts.len;
        const bool cut = valid && pos == (REV ? cuts.T - 1 : 0);
        V start = vzero<V>();
        if (cuts.stage != nullptr && cut) start = Tr::load1(cuts.stage + (row - cuts.first_row));
        t[e] = vselect(cut, vfma(g[e], start, t[e]), t[e]);
        g[e] = vselect(cut, vzero<V>(), g[e]);
        if (++pos == cuts.T) {
            pos = 0;
            ++row;
        }
    }
}

// Backward scan: `after[e]` is the gate that follows element e in its row and
// `before[e]` the state that precedes it; at a row's last element nothing
// follows (0), at its first the state before it is the row's initial state.
// is_first[e] / row_of[e] tell the caller where to put the gradient of that
// initial state.
template <class Tr>
__device__ __forceinline__ void cut_rows_backward(typename Tr::V (&after)[Tr::EPV], typename Tr::V (&before)[Tr::EPV],
                                                  bool (&is_first)[Tr::EPV], int (&row_of)[Tr::EPV], int rel0,
                                                  const Cuts<Tr>& cuts) {
    using V = typename Tr::V;
    int row, pos;
    split_position(rel0, cuts.T, cuts.inv_T, row, pos);
#pragma unroll
    for (int e = 0; e < Tr::EPV; ++e) {
        const bool valid = (unsigned)(rel0 + e) < (unsigned)cuts.len;
        const bool first = valid && pos == 0;
        const bool last = valid && pos == cuts.T - 1;
        V start = vzero<V>();
        if (cuts.stage != nullptr && first) start = Tr::load1(cuts.stage + (row - cuts.first_row));
        before[e] = vselect(first, start, before[e]);
        after[e] = vselect(last, vzero<V>(), after[e]);
        is_first[e] = first;
        row_of[e] = row;
        if (++pos == cuts.T) {
            pos = 0;
            ++row;
        }
    }
}

// Stages the initial states of the rows that the sub-tile [sub_rel, sub_rel+sub)
// touches (positions relative to the group) into the wave's LDS area.
template <class Tr>
__device__ __forceinline__ Cuts<Tr> stage_row_starts(const typename Tr::S* __restrict__ initial_of_group, int T,
                                                     int len, int sub_rel, int sub, typename Tr::S* stage, int lane) {
    Cuts<Tr> cuts;
    cuts.T = T;
    cuts.inv_T = 1.0f / (float)T;
    cuts.len = len;
    cuts.first_row = 0;
    cuts.stage = nullptr;
    if (initial_of_group != nullptr) {
        const int rel_first = sub_rel > 0 ? sub_rel : 0;
        const int rel_last = sub_rel + sub - 1 < len - 1 ? sub_rel + sub - 1 : len - 1;
        if (rel_first <= rel_last) {  // wave-uniform
            cuts.first_row = rel_first / T;
            const int count = rel_last / T - cuts.first_row + 1;  // at most `sub`
            for (int i = lane; i < count; i += 64) stage[i] = initial_of_group[cuts.first_row + i];
        }
        cuts.stage = stage;
        __syncthreads();  // makes the staged values visible to the other lanes
    }
    return cuts;
}

// ---------------------------------------------------------------------------
// Forward kernel (REV = false) and plain reverse scan (REV = true).
// A workgroup holds R rows x W waves per row (R = blockDim.x / 64 / W); the
// rows of a workgroup are adjacent in memory, so with W*R = 16 one tile step
// of the workgroup covers one contiguous span of 16 sub-tiles.
// ---------------------------------------------------------------------------
template <class Tr, int W, int U, bool REV, bool ALIGNED, bool REGULAR, bool SPLIT, int ACT, bool PACKED>
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

    const int lane = threadIdx.x & 63;
    // Packed rows: this workgroup scans rows [first_row, first_row + nrows) as one row of `len` elements.
    const int64_t first_row = PACKED ? (int64_t)blockIdx.x * group : 0;
    const int64_t len = PACKED ? (rows - first_row < group ? rows - first_row : (int64_t)group) * T : T;
    const int64_t longest = PACKED ? (int64_t)group * T : T;
    // rows start at the same misalignment when their length is a multiple of the grid spacing
    const int head = REGULAR ? 0 : (ALIGNED ? (longest % G == 0 ? row_lead<Tr>(gates, G) : G - 1) : 0);
    const int64_t ntiles = tiles_per_row(longest, TILE, head);
    __shared__ V slots_all[W == 1 ? 1 : 2 * kSlotsPerBuffer];
    __shared__ S stage_all[PACKED ? W * SUB : 1];
    // Split rows: the workgroups take tiles by ticket, row by row, until none
    // is left; a workgroup only ever waits for tiles whose owners started before it.
    __shared__ long long split_mailbox[2];
    SplitWalk walk;  // starts at row blockIdx % rows
    walk.row = SPLIT ? (int64_t)(blockIdx.x % rows) : 0;
    walk.has_drawn = false;
    for (bool first_visit = true;; first_visit = false) {
    int64_t row;
    int w, slot_base;
    int64_t k_begin = 0, k_end = ntiles;
    if constexpr (SPLIT) {
        if (!take_split_tile(split, rows, ntiles, walk, row, k_begin, split_mailbox)) break;
        k_end = k_begin + 1;
        w = threadIdx.x >> 6;
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

    const int64_t lo = (ALIGNED && !REGULAR) ? row_lead<Tr>(gates + row * T, G) : 0;
    const int64_t hi = lo + len;
    const S* __restrict__ grow = gates + row * T - lo;
    const typename Tr::TokS* __restrict__ trow = tokens + row * T - lo;
    S* __restrict__ orow = out + row * T - lo;

    // state the row starts from (one element per row; absent = zero); a split
    // row needs it in its first tile only; packed rows take theirs at the cuts
    const V row_start =
        (!PACKED && initial != nullptr && (!SPLIT || k_begin == 0)) ? Tr::load1(initial + row) : vzero<V>();
    V carry = row_start;

    // Position of this wave's sub-tile in tile step k.
    auto sub_tile_base = [&](int64_t k) {
        const int64_t tile = REV ? (ntiles - 1 - k) : k;
        return tile * TILE + (int64_t)(REV ? (W - 1 - w) : w) * SUB;
    };
    // One tile step of this wave.  FULL (a compile-time flag) says that the
    // wave's sub-tile lies entirely inside the row: that copy of the body has no
    // masking code.  The other copy serves the (at most two) ragged tiles of a
    // row; it exists only in the kernels for arbitrary row starts and lengths.
    auto tile_step = [&](int64_t k, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
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
#pragma unroll
        for (int j = 0; j < U; ++j) {
            V g[EPV], t[EPV];
            Tr::unpack(graw[j], g);
            activate<ACT>(g);
            Tr::unpack(traw[j], t);
            if constexpr (PACKED) cut_rows<Tr, REV>(g, t, (int)(sub_base - lo) + vec_offset<U, EPV, REV>(j, lane), cuts);
            constexpr int e0 = REV ? EPV - 1 : 0;
            V A = g[e0];
            V X = t[e0];
#pragma unroll
            for (int i = 1; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                X = vfma(g[e], X, t[e]);
                A = vmul(A, g[e]);
            }
            wave_scan_inclusive(A, X);
            totA[j] = read_lane<63>(A);
            totX[j] = read_lane<63>(X);
            exA[j] = shift_up1(A, vone<V>());
            exX[j] = shift_up1(X, vzero<V>());
        }

        V c;
        if constexpr (SPLIT) {
            exchange_carries_split<V, W, U>(totA, totX, c, slots, w, lane, split, split_records(split, rows) + row * ntiles, 1, k,
                                            row_start);
        } else {
            exchange_carries<V, W, U>(totA, totX, carry, c, slots, (int)(k & 1), w, lane);
        }

        // Pass 2: the plain recurrence from the state entering each lane.
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if constexpr (Tr::kNarrow) {
                forget_unpacked(graw[j]);
                forget_unpacked(traw[j]);
            }
            V g[EPV], t[EPV];
            Tr::unpack(graw[j], g);
            activate<ACT>(g);
            Tr::unpack(traw[j], t);
            if constexpr (PACKED) cut_rows<Tr, REV>(g, t, (int)(sub_base - lo) + vec_offset<U, EPV, REV>(j, lane), cuts);
            V x = vfma(exA[j], c, exX[j]);  // state entering this lane's vector
            c = vfma(totA[j], c, totX[j]);  // state entering the next block
            V o[EPV];
#pragma unroll
            for (int i = 0; i < EPV; ++i) {
                const int e = REV ? EPV - 1 - i : i;
                x = vfma(g[e], x, t[e]);
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

// ---------------------------------------------------------------------------
// Fused backward kernel: reverse-time scan over gate[t+1] producing d_tokens,
// and d_gates[t] = d_tokens[t] * conj(x[t-1]) in the same pass.
// ---------------------------------------------------------------------------
template <class Tr, int W, int U, bool ALIGNED, bool REGULAR, bool SPLIT, int ACT, bool PACKED>
__global__ void __launch_bounds__(64 * kMaxWavesPerBlock)
    scan_backward_kernel(const typename Tr::S* __restrict__ gates, const typename Tr::S* __restrict__ states,
                         const typename Tr::S* __restrict__ grad_out, typename Tr::S* __restrict__ d_gates,
                         typename Tr::TokS* __restrict__ d_tokens, int64_t rows, int64_t T, SplitHeader* split,
                         const typename Tr::S* __restrict__ initial, typename Tr::S* __restrict__ d_initial, int G,
                         int group) {
    using S = typename Tr::S;
    using V = typename Tr::V;
    constexpr int EPV = Tr::EPV;
    constexpr int64_t SUB = (int64_t)U * 64 * EPV;
    constexpr int64_t TILE = SUB * W;
    static_assert(!PACKED || (!SPLIT && !REGULAR), "packed rows use the general kernels, one group per workgroup");

    const int lane = threadIdx.x & 63;
    // Packed rows: this workgroup scans rows [first_row, first_row + nrows) as one row of `len` elements.
    const int64_t first_row = PACKED ? (int64_t)blockIdx.x * group : 0;
    const int64_t len = PACKED ? (rows - first_row < group ? rows - first_row : (int64_t)group) * T : T;
    const int64_t longest = PACKED ? (int64_t)group * T : T;
    // rows start at the same misalignment when their length is a multiple of the grid spacing
    const int head = REGULAR ? 0 : (ALIGNED ? (longest % G == 0 ? row_lead<Tr>(gates, G) : G - 1) : 0);
    const int64_t ntiles = tiles_per_row(longest, TILE, head);
    __shared__ V slots_all[W == 1 ? 1 : 2 * kSlotsPerBuffer];
    __shared__ S stage_all[PACKED ? W * SUB : 1];
    // Split rows: the workgroups take tiles by ticket, row by row, until none
    // is left; a workgroup only ever waits for tiles whose owners started before it.
    __shared__ long long split_mailbox[2];
    SplitWalk walk;  // starts at row blockIdx % rows
    walk.row = SPLIT ? (int64_t)(blockIdx.x % rows) : 0;
    walk.has_drawn = false;
    for (bool first_visit = true;; first_visit = false) {
    int64_t row;
    int w, slot_base;
    int64_t k_begin = 0, k_end = ntiles;
    if constexpr (SPLIT) {
        if (!take_split_tile(split, rows, ntiles, walk, row, k_begin, split_mailbox)) break;
        k_end = k_begin + 1;
        w = threadIdx.x >> 6;
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

    const int64_t lo = (ALIGNED && !REGULAR) ? row_lead<Tr>(gates + row * T, G) : 0;
    const int64_t hi = lo + len;
    const S* __restrict__ arow = gates + row * T - lo;
    const S* __restrict__ xrow = states + row * T - lo;
    const S* __restrict__ drow = grad_out + row * T - lo;
    S* __restrict__ dgrow = d_gates + row * T - lo;
    typename Tr::TokS* __restrict__ dtrow = d_tokens + row * T - lo;

    V carry = vzero<V>();

    // Gradient of x[-1], conj(gate[0]) * g[0], from g at position 0 of the row's
    // first tile.  Positions below the row's first element (position lo) carry
    // gate 1 and grad_out 0, so with lo > 0 that g already is the gradient;
    // with lo == 0 the last factor is still missing.
    auto store_start_gradient = [&](V g_low) {
        if (lo == 0) g_low = vmul(vconj(activate1<ACT>(Tr::load1(arow))), g_low);
        if (lane == 0) Tr::store1(d_initial + row, g_low);
    };

    // Position of this wave's sub-tile in tile step k (reverse time).
    auto sub_tile_base = [&](int64_t k) {
        const int64_t tile = ntiles - 1 - k;
        return tile * TILE + (int64_t)(W - 1 - w) * SUB;
    };
    // One tile step of this wave; FULL as in the forward kernel.
    auto tile_step = [&](int64_t k, auto full_tag) {
        constexpr bool FULL = decltype(full_tag)::value;
        const int64_t sub_base = sub_tile_base(k);
        const int64_t sub_end = sub_base + SUB;
        const Window win = make_window(lo, hi, sub_base);
        const bool touches = FULL || (win.hi > 0 && win.lo < SUB);  // wave-uniform
        const S* __restrict__ asub = arow + sub_base;
        const S* __restrict__ dsub = drow + sub_base;
        const S* __restrict__ xsub = xrow + sub_base;
        S* __restrict__ dgsub = dgrow + sub_base;
        typename Tr::TokS* __restrict__ dtsub = dtrow + sub_base;

        // x[-1], the state the forward scan started from (absent = zero), is
        // needed by the sub-tile that holds the row's first element
        V x_start = vzero<V>();
        if (!PACKED && initial != nullptr && sub_base <= lo && lo < sub_end) x_start = Tr::load1(initial + row);  // wave-uniform
        Cuts<Tr> cuts;  // packed rows take their initial states at the cuts instead
        if constexpr (PACKED) {
            cuts = stage_row_starts<Tr>(initial != nullptr ? initial + first_row : nullptr, (int)T, (int)len,
                                        (int)(sub_base - lo), (int)SUB, stage_all + w * SUB, lane);
        }

        u32x4_t araw[U], draw[U], xraw[U];
        if (touches) {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                const int off = vec_offset<U, EPV, true>(j, lane);
                araw[j] = load_raw<Tr, ALIGNED, FULL>(asub, off, win, identity_gate<ACT, V>());
                draw[j] = load_raw<Tr, ALIGNED, FULL>(dsub, off, win, vzero<V>());
                xraw[j] = load_raw<Tr, ALIGNED, FULL>(xsub, off, win, x_start);
            }
        } else {
#pragma unroll
            for (int j = 0; j < U; ++j) {
                araw[j] = fill_raw<Tr>(identity_gate<ACT, V>());
                draw[j] = fill_raw<Tr>(vzero<V>());
                xraw[j] = fill_raw<Tr>(x_start);
            }
        }

        // The two elements just outside the sub-tile: gate at sub_end and x at
        // sub_base-1.  Addresses are clamped into the row so the loads are
        // unconditional; out-of-row positions take the identity gate and x[-1].
        V a_edge, x_edge;
        {
            const int64_t ia = sub_end < hi ? (sub_end > lo ? sub_end : lo) : hi - 1;
            int64_t ix = sub_base - 1;
            ix = ix < lo ? lo : (ix < hi ? ix : hi - 1);
            const V av = activate1<ACT>(Tr::load1(arow + ia));
            const V xv = Tr::load1(xrow + ix);
            a_edge = vselect(sub_end >= lo && sub_end < hi, av, vone<V>());
            x_edge = vselect(sub_base - 1 >= lo && sub_base - 1 < hi, xv, x_start);
        }

        // Pass 1.  Gates are needed one element later (gate[t+1]) and states one
        // element earlier (x[t-1]).  In scan order the vector at the next higher
        // address belongs to lane-1 and the one at the next lower address to
        // lane+1, so each block needs one value from each neighbour: a_next (the
        // first gate of the vector above) and x_prev (the last state of the
        // vector below).
        V a_next[U], x_prev[U];
        V totA[U], totX[U], exA[U], exX[U];
#pragma unroll
        for (int j = 0; j < U; ++j) {
            V a[EPV], d[EPV], x[EPV];
            Tr::unpack(araw[j], a);
            activate<ACT>(a);
            Tr::unpack(draw[j], d);
            Tr::unpack(xraw[j], x);
            V hi_edge, lo_edge;
            if (j == 0) {
                hi_edge = a_edge;
            } else {
                V above[EPV];
                Tr::unpack(araw[j > 0 ? j - 1 : 0], above);
                hi_edge = read_lane<63>(activate1<ACT>(above[0]));
            }
            if (j == U - 1) {
                lo_edge = x_edge;
            } else {
                V below[EPV];
                Tr::unpack(xraw[j < U - 1 ? j + 1 : j], below);
                lo_edge = read_lane<0>(below[EPV - 1]);
            }
            a_next[j] = shift_up1(a[0], hi_edge);
            x_prev[j] = shift_down1(x[EPV - 1], lo_edge);

            // after[e]: the gate that follows element e; before[e]: the state that precedes it
            V after[EPV], before[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                after[e] = e < EPV - 1 ? a[e + 1] : a_next[j];
                before[e] = e > 0 ? x[e - 1] : x_prev[j];
            }
            if constexpr (PACKED) {
                bool is_first[EPV];
                int row_of[EPV];
                cut_rows_backward<Tr>(after, before, is_first, row_of,
                                      (int)(sub_base - lo) + vec_offset<U, EPV, true>(j, lane), cuts);
            }
            V A = vconj(after[EPV - 1]);
            V X = d[EPV - 1];
#pragma unroll
            for (int e = EPV - 2; e >= 0; --e) {
                const V ga = vconj(after[e]);
                X = vfma(ga, X, d[e]);
                A = vmul(A, ga);
            }
            wave_scan_inclusive(A, X);
            totA[j] = read_lane<63>(A);
            totX[j] = read_lane<63>(X);
            exA[j] = shift_up1(A, vone<V>());
            exX[j] = shift_up1(X, vzero<V>());
        }

        V c;
        if constexpr (SPLIT) {
            exchange_carries_split<V, W, U>(totA, totX, c, slots, w, lane, split, split_records(split, rows) + row * ntiles, 1, k,
                                            vzero<V>());
        } else {
            exchange_carries<V, W, U>(totA, totX, carry, c, slots, (int)(k & 1), w, lane);
        }
        // Pass 2: the plain reverse recurrence and the gate gradient.
#pragma unroll
        for (int j = 0; j < U; ++j) {
            if constexpr (Tr::kNarrow) {
                forget_unpacked(araw[j]);
                forget_unpacked(draw[j]);
                forget_unpacked(xraw[j]);
            }
            V a[EPV], d[EPV], x[EPV];
            Tr::unpack(araw[j], a);
            activate<ACT>(a);
            Tr::unpack(draw[j], d);
            Tr::unpack(xraw[j], x);
            V gr = vfma(exA[j], c, exX[j]);  // g entering this lane's vector from above
            c = vfma(totA[j], c, totX[j]);
            const int off = vec_offset<U, EPV, true>(j, lane);
            V after[EPV], before[EPV];
#pragma unroll
            for (int e = 0; e < EPV; ++e) {
                after[e] = e < EPV - 1 ? a[e + 1] : a_next[j];
                before[e] = e > 0 ? x[e - 1] : x_prev[j];
            }
            bool is_first[EPV];
            int row_of[EPV];
            if constexpr (PACKED) {
                cut_rows_backward<Tr>(after, before, is_first, row_of, (int)(sub_base - lo) + off, cuts);
            }
            V dt[EPV], dg[EPV];
#pragma unroll
            for (int e = EPV - 1; e >= 0; --e) {
                gr = vfma(vconj(after[e]), gr, d[e]);
                dt[e] = gr;
                dg[e] = vmul(gr, vconj(before[e]));
                if constexpr (ACT != kGateIdentity) dg[e] = vmul(dg[e], gate_slope<ACT>(a[e]));
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
                        if (is_first[e]) Tr::store1(d_initial + first_row + row_of[e], vmul(vconj(a[e]), dt[e]));
                    }
                }
            }
        }

        // A split row's last tile step ends at the row's first element: after
        // pass 2, c is g at the lowest position of this wave's sub-tile.
        if constexpr (SPLIT) {
            if (d_initial != nullptr && k == ntiles - 1 && w == W - 1) store_start_gradient(c);  // wave-uniform
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
    // after the last tile step the carry is g at position 0 of the first tile
    if constexpr (!SPLIT && !PACKED) {
        if (d_initial != nullptr && w == 0) store_start_gradient(carry);  // wave-uniform
    }
    }  // visits
}

// ---------------------------------------------------------------------------
// Host side.
// ---------------------------------------------------------------------------
thread_local int g_last_hip_error = 0;

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
// along one row it reaches the 5.7-6.1 TB/s of a plain linear sweep.  So a row
// gets as many waves as it has sub-tiles (up to 16).  Short rows keep small
// workgroups (256 threads, several rows each): packing more short rows into
// one large workgroup measured slower.
Plan choose_plan(int64_t T, int64_t sub, int64_t element_bytes) {
    const Plan& forced = forced_plan();
    // one wave per 4 KiB of row, but never more waves than sub-tiles
    int w = 1;
    while (w < kMaxWavesPerBlock && (int64_t)w * 4096 < T * element_bytes && (int64_t)w * sub < T) w *= 2;
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

int launch_status(hipError_t e) {
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ASCAN_ERR_LAUNCH;
    }
    return ASCAN_OK;
}

template <class Tr, int W, bool REV, bool ALIGNED, bool REGULAR, int ACT>
hipError_t launch_forward(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                          int64_t T, int grid, int rows_per_block, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? Tuning<Tr>::U : Tuning<Tr>::UG;
    const unsigned blocks = (unsigned)((rows + rows_per_block - 1) / rows_per_block);
    const unsigned threads = 64u * W * rows_per_block;
    return launch(scan_forward_kernel<Tr, W, U, REV, ALIGNED, REGULAR, false, ACT, false>, blocks, threads, stream,
                  static_cast<const S*>(gates), static_cast<const TokS*>(tokens), static_cast<S*>(out), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial), grid, 0);
}

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

// Caller-provided table for split rows (may be absent).
struct Workspace {
    void* ptr;
    size_t bytes;
};

// Split-row policy.  A call is split when its rows alone would leave most
// compute units without a workgroup and every row has several tiles.  Split
// tiles are small (4 waves) so that several workgroups share a compute unit
// and overlap each other's loads, waits and stores.
constexpr int kSplitWaves = 4;
constexpr int64_t kSplitMaxRowsDefault = 128;

int64_t split_max_rows() {
    static const int64_t v = [] {
        const char* s = getenv("ASCAN_SPLIT_MAX_ROWS");
        return s ? (int64_t)atoll(s) : kSplitMaxRowsDefault;
    }();
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

bool want_split(int64_t rows, int64_t ntiles) { return rows <= split_max_rows() && ntiles >= 8; }

size_t split_bytes(int64_t rows, int64_t ntiles) {
    return sizeof(SplitHeader) + (size_t)rows * sizeof(SplitTicket) +
           (size_t)rows * (size_t)ntiles * sizeof(SplitRecord);
}

bool workspace_fits(const Workspace& ws, int64_t rows, int64_t ntiles) {
    return ws.ptr != nullptr && (reinterpret_cast<uintptr_t>(ws.ptr) % alignof(SplitRecord)) == 0 &&
           ws.bytes >= split_bytes(rows, ntiles);
}

hipError_t reset_split_table(const Workspace& ws, int64_t rows, int64_t ntiles, hipStream_t stream) {
    const size_t nwords = split_bytes(rows, ntiles) / sizeof(uint32_t);
    const unsigned blocks = (unsigned)((nwords + 255) / 256);
    return launch(split_reset_kernel, blocks, 256u, stream, static_cast<uint32_t*>(ws.ptr), nwords,
                  split_wait_limit());
}

// Number of workgroups of `kernel` (of `threads` threads, no dynamic LDS) the
// current device holds at one time.  Queried once per kernel and device.
template <class K>
unsigned resident_workgroups(K kernel, int threads) {
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
        known = (unsigned)per_cu * (unsigned)cus;
        cache[device].store(known, std::memory_order_relaxed);
    }
    return known;
}

// Tiles per row as the kernels count them (tiles_per_row on the device).
template <class Tr>
int64_t host_tiles_per_row(int64_t T, int64_t tile, bool regular, const Lead& at) {
    const int head = regular ? 0 : (T % at.grid == 0 ? at.lead : at.grid - 1);
    return (T + head + tile - 1) / tile;
}

template <class Tr, bool REV, bool REGULAR, int ACT>
hipError_t launch_forward_split(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                                int64_t T, int grid, int64_t ntiles, const Workspace& ws, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? Tuning<Tr>::U : Tuning<Tr>::UG;
    auto kernel = scan_forward_kernel<Tr, kSplitWaves, U, REV, true, REGULAR, true, ACT, false>;
    const unsigned resident = resident_workgroups(kernel, 64 * kSplitWaves);
    if (resident == 0) return hipErrorInvalidConfiguration;
    const hipError_t e = reset_split_table(ws, rows, ntiles, stream);
    if (e != hipSuccess) return e;
    const int64_t tiles = rows * ntiles;
    return launch(kernel, (unsigned)(tiles < resident ? tiles : resident), 64u * kSplitWaves, stream,
                  static_cast<const S*>(gates), static_cast<const TokS*>(tokens), static_cast<S*>(out), rows, T,
                  static_cast<SplitHeader*>(ws.ptr), static_cast<const S*>(initial), grid, 0);
}

template <class Tr, bool REGULAR, int ACT>
hipError_t launch_backward_split(const void* gates, const void* states, const void* grad_out, void* d_gates,
                                 void* d_tokens, const void* initial, void* d_initial, int64_t rows, int64_t T,
                                 int grid, int64_t ntiles, const Workspace& ws, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    constexpr int U = REGULAR ? Tuning<Tr>::UB : Tuning<Tr>::UBG;
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

// Packed-row policy.  Rows shorter than kPackedMaxRowBytes (of states) are
// scanned in groups, one group per 4-wave workgroup; a group fills one tile of
// the general kernel, counting the lead of its first element, and when possible
// is a whole number of 128-byte lines long so that every group starts on the
// grid like the first.  ASCAN_PACKED_MAX_ROW_BYTES overrides the limit (0
// switches packing off), read once.
constexpr int kPackedWaves = 4;
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
    const int64_t whole_lines = grid / gcd64(T, grid);  // rows per whole number of grid cells
    if (group >= whole_lines) group -= group % whole_lines;
    return (int)group;
}

template <class Tr, bool REV, bool ALIGNED, int ACT>
hipError_t launch_forward_packed(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                                 int64_t T, int grid, int group, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    const unsigned blocks = (unsigned)((rows + group - 1) / group);
    return launch(scan_forward_kernel<Tr, kPackedWaves, Tuning<Tr>::UG, REV, ALIGNED, false, false, ACT, true>, blocks,
                  64u * kPackedWaves, stream, static_cast<const S*>(gates), static_cast<const TokS*>(tokens),
                  static_cast<S*>(out), rows, T, static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial),
                  grid, group);
}

template <class Tr, bool ALIGNED, int ACT>
hipError_t launch_backward_packed(const void* gates, const void* states, const void* grad_out, void* d_gates,
                                  void* d_tokens, const void* initial, void* d_initial, int64_t rows, int64_t T,
                                  int grid, int group, hipStream_t stream) {
    using S = typename Tr::S;
    using TokS = typename Tr::TokS;
    const unsigned blocks = (unsigned)((rows + group - 1) / group);
    return launch(scan_backward_kernel<Tr, kPackedWaves, Tuning<Tr>::UBG, ALIGNED, false, false, ACT, true>, blocks,
                  64u * kPackedWaves, stream, static_cast<const S*>(gates), static_cast<const S*>(states),
                  static_cast<const S*>(grad_out), static_cast<S*>(d_gates), static_cast<TokS*>(d_tokens), rows, T,
                  static_cast<SplitHeader*>(nullptr), static_cast<const S*>(initial), static_cast<S*>(d_initial), grid,
                  group);
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

// Kernels with the sigmoid gate exist for the real dtypes, forward in time.
template <class Tr>
constexpr bool kHasSigmoid = std::is_same<typename Tr::V, float>::value;

template <class Tr>
int forward_typed(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows, int64_t T,
                  bool reverse, int act, const Workspace& ws, hipStream_t stream) {
    constexpr int64_t kElem = (int64_t)sizeof(typename Tr::S);
    constexpr int64_t SUB = (int64_t)Tuning<Tr>::U * 64 * Tr::EPV;    // regular kernels
    constexpr int64_t SUBG = (int64_t)Tuning<Tr>::UG * 64 * Tr::EPV;  // kernels with masking code
    Plan plan = choose_plan(T, SUB, kElem);
    const void* const state_like[] = {gates, out};
    const Lead at = find_lead<Tr>(state_like, tokens);
    const bool same_lead = at.same;
    const int lead = at.lead;
    const Access access = choose_access(same_lead, lead, T, SUB * plan.waves_per_row);
    if (access != Access::kRegular) plan = choose_plan(T, SUBG, kElem);
    const int R = plan.rows_per_block;
    hipError_t err = hipSuccess;
    if (const int group = packed_group(rows, T, kElem, SUBG * kPackedWaves, same_lead ? at.grid : 1)) {
#define ASCAN_FWD_PACKED(REV, AL, ACT) \
    launch_forward_packed<Tr, REV, AL, ACT>(gates, tokens, out, initial, rows, T, at.grid, group, stream)
        if (act == kGateSigmoid) {
            if constexpr (kHasSigmoid<Tr>) {
                err = same_lead ? ASCAN_FWD_PACKED(false, true, kGateSigmoid) : ASCAN_FWD_PACKED(false, false, kGateSigmoid);
            }
        } else if (same_lead) {
            err = reverse ? ASCAN_FWD_PACKED(true, true, kGateIdentity) : ASCAN_FWD_PACKED(false, true, kGateIdentity);
        } else {
            err = reverse ? ASCAN_FWD_PACKED(true, false, kGateIdentity) : ASCAN_FWD_PACKED(false, false, kGateIdentity);
        }
#undef ASCAN_FWD_PACKED
        return launch_status(err);
    }
    if (same_lead && ws.ptr != nullptr) {
        const bool regular = lead == 0 && T % (SUB * kSplitWaves) == 0;
        const int64_t ntiles = host_tiles_per_row<Tr>(T, (regular ? SUB : SUBG) * kSplitWaves, regular, at);
        if (want_split(rows, ntiles) && workspace_fits(ws, rows, ntiles)) {
#define ASCAN_FWD_SPLIT(REV, REG, ACT) \
    launch_forward_split<Tr, REV, REG, ACT>(gates, tokens, out, initial, rows, T, at.grid, ntiles, ws, stream)
            if (act == kGateSigmoid) {
                if constexpr (kHasSigmoid<Tr>) {
                    err = regular ? ASCAN_FWD_SPLIT(false, true, kGateSigmoid) : ASCAN_FWD_SPLIT(false, false, kGateSigmoid);
                }
            } else if (regular) {
                err = reverse ? ASCAN_FWD_SPLIT(true, true, kGateIdentity) : ASCAN_FWD_SPLIT(false, true, kGateIdentity);
            } else {
                err = reverse ? ASCAN_FWD_SPLIT(true, false, kGateIdentity) : ASCAN_FWD_SPLIT(false, false, kGateIdentity);
            }
#undef ASCAN_FWD_SPLIT
            return launch_status(err);
        }
    }
#define ASCAN_FWD_ARGS gates, tokens, out, initial, rows, T, at.grid, R, stream
#define ASCAN_FWD(WV, AL, REG)                                                                  \
    do {                                                                                        \
        if (act == kGateSigmoid) {                                                              \
            if constexpr (kHasSigmoid<Tr>)                                                      \
                err = launch_forward<Tr, WV, false, AL, REG, kGateSigmoid>(ASCAN_FWD_ARGS);     \
        } else if (reverse) {                                                                   \
            err = launch_forward<Tr, WV, true, AL, REG, kGateIdentity>(ASCAN_FWD_ARGS);         \
        } else {                                                                                \
            err = launch_forward<Tr, WV, false, AL, REG, kGateIdentity>(ASCAN_FWD_ARGS);        \
        }                                                                                       \
    } while (0)
#define ASCAN_FWD_W(AL, REG)                            \
    switch (plan.waves_per_row) {                       \
        case 1: ASCAN_FWD(1, AL, REG); break;           \
        case 2: ASCAN_FWD(2, AL, REG); break;           \
        case 4: ASCAN_FWD(4, AL, REG); break;           \
        case 8: ASCAN_FWD(8, AL, REG); break;           \
        default: ASCAN_FWD(16, AL, REG); break;         \
    }
    if (access == Access::kRegular) {
        ASCAN_FWD_W(true, true);
    } else if (access == Access::kVector) {
        ASCAN_FWD_W(true, false);
    } else {
        ASCAN_FWD_W(false, false);
    }
#undef ASCAN_FWD_W
#undef ASCAN_FWD
#undef ASCAN_FWD_ARGS
    return launch_status(err);
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
    Plan plan = choose_plan(T, SUB, kElem);
    const Access access = choose_access(same_lead, lead, T, SUB * plan.waves_per_row);
    if (access != Access::kRegular) plan = choose_plan(T, SUBG, kElem);
    const int R = plan.rows_per_block;
    hipError_t err = hipSuccess;
    if (const int group = packed_group(rows, T, kElem, SUBG * kPackedWaves, same_lead ? at.grid : 1)) {
#define ASCAN_BWD_PACKED(AL, ACT)                                                                                  \
    launch_backward_packed<Tr, AL, ACT>(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows, T, \
                                        at.grid, group, stream)
        if (act == kGateSigmoid) {
            if constexpr (kHasSigmoid<Tr>) {
                err = same_lead ? ASCAN_BWD_PACKED(true, kGateSigmoid) : ASCAN_BWD_PACKED(false, kGateSigmoid);
            }
        } else {
            err = same_lead ? ASCAN_BWD_PACKED(true, kGateIdentity) : ASCAN_BWD_PACKED(false, kGateIdentity);
        }
#undef ASCAN_BWD_PACKED
        return launch_status(err);
    }
    if (same_lead && ws.ptr != nullptr) {
        const bool regular = lead == 0 && T % (SUB * kSplitWaves) == 0;
        const int64_t ntiles = host_tiles_per_row<Tr>(T, (regular ? SUB : SUBG) * kSplitWaves, regular, at);
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

size_t element_size(int dtype) {
    switch (dtype) {
        case ASCAN_F32: return 4;
        case ASCAN_BF16: return 2;
        case ASCAN_F16: return 2;
        case ASCAN_C64: return 8;
        case ASCAN_C64_REAL_TOKENS: return 8;
        default: return 0;
    }
}

// Element size of tokens / d_tokens.
size_t token_size(int dtype) { return dtype == ASCAN_C64_REAL_TOKENS ? 4 : element_size(dtype); }

bool element_aligned(const void* p, size_t es) { return (reinterpret_cast<uintptr_t>(p) % es) == 0; }

// Largest row count one launch can address: gridDim.x is limited to 2^31-1.
constexpr int64_t kMaxBlocks = 2147483647LL;

// Calls fn with a value of the traits type that `dtype` selects.
template <class Fn>
int with_traits(int dtype, Fn fn) {
    switch (dtype) {
        case ASCAN_F32: return fn(TraitsF32{});
        case ASCAN_BF16: return fn(TraitsBF16{});
        case ASCAN_F16: return fn(TraitsF16{});
        case ASCAN_C64: return fn(TraitsC64{});
        default: return fn(TraitsC64RealTokens{});
    }
}

bool activation_supported(int act, int dtype, bool reverse) {
    if (act == kGateIdentity) return true;
    return act == kGateSigmoid && !reverse && (dtype == ASCAN_F32 || dtype == ASCAN_BF16 || dtype == ASCAN_F16);
}

int forward_checked(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                    int64_t seqlen, int dtype, int reverse, int act, const Workspace& ws, void* stream) {
    const size_t es = element_size(dtype);
    if (es == 0) return ASCAN_ERR_BAD_DTYPE;
    if (!activation_supported(act, dtype, reverse != 0)) return ASCAN_ERR_BAD_ACTIVATION;
    if (rows < 0 || seqlen < 0 || rows > kMaxBlocks) return ASCAN_ERR_BAD_SHAPE;
    if (rows == 0 || seqlen == 0) return ASCAN_OK;
    if (!gates || !tokens || !out) return ASCAN_ERR_NULL_POINTER;
    if (!element_aligned(gates, es) || !element_aligned(tokens, token_size(dtype)) || !element_aligned(out, es) ||
        !element_aligned(initial, es))
        return ASCAN_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return with_traits(dtype, [&](auto traits) {
        return forward_typed<decltype(traits)>(gates, tokens, out, initial, rows, seqlen, reverse != 0, act, ws, s);
    });
}

int backward_checked(const void* gates, const void* states, const void* grad_out, void* d_gates, void* d_tokens,
                     const void* initial, void* d_initial, int64_t rows, int64_t seqlen, int dtype, int act,
                     const Workspace& ws, void* stream) {
    const size_t es = element_size(dtype);
    if (es == 0) return ASCAN_ERR_BAD_DTYPE;
    if (!activation_supported(act, dtype, false)) return ASCAN_ERR_BAD_ACTIVATION;
    if (rows < 0 || seqlen < 0 || rows > kMaxBlocks) return ASCAN_ERR_BAD_SHAPE;
    if (rows == 0 || seqlen == 0) return ASCAN_OK;
    if (!gates || !states || !grad_out || !d_gates || !d_tokens) return ASCAN_ERR_NULL_POINTER;
    if (!element_aligned(gates, es) || !element_aligned(states, es) || !element_aligned(grad_out, es) ||
        !element_aligned(d_gates, es) || !element_aligned(d_tokens, token_size(dtype)) ||
        !element_aligned(initial, es) || !element_aligned(d_initial, es))
        return ASCAN_ERR_MISALIGNED;
    hipStream_t s = static_cast<hipStream_t>(stream);
    return with_traits(dtype, [&](auto traits) {
        return backward_typed<decltype(traits)>(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows,
                                                seqlen, act, ws, s);
    });
}

}  // namespace

extern "C" {

int ascan_forward(const void* gates, const void* tokens, void* out, int64_t rows, int64_t seqlen, int dtype,
                  int reverse, void* stream) {
    return forward_checked(gates, tokens, out, nullptr, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY,
                           Workspace{nullptr, 0}, stream);
}

int ascan_backward(const void* gates, const void* states, const void* grad_out, void* d_gates, void* d_tokens,
                   int64_t rows, int64_t seqlen, int dtype, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, nullptr, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, Workspace{nullptr, 0}, stream);
}

size_t ascan_workspace_bytes(int64_t rows, int64_t seqlen, int dtype) {
    const size_t es = element_size(dtype);
    if (es == 0 || rows <= 0 || seqlen <= 0) return 0;
    // the smallest split tile any kernel uses for this dtype: 4 waves x 2 blocks x 64 vectors
    const int64_t epv = 16 / (int64_t)es;
    const int64_t tile = (int64_t)kSplitWaves * 2 * 64 * epv;
    // rows are addressed from the 128-byte boundary below their first element at most
    const int64_t head = 128 / (int64_t)es - 1;
    const int64_t ntiles = (seqlen + head + tile - 1) / tile;
    if (!want_split(rows, ntiles) || rows * ntiles > 2147483647LL) return 0;
    return split_bytes(rows, ntiles);
}

int ascan_forward_split(const void* gates, const void* tokens, void* out, int64_t rows, int64_t seqlen, int dtype,
                        int reverse, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_checked(gates, tokens, out, nullptr, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY,
                           Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_split(const void* gates, const void* states, const void* grad_out, void* d_gates,
                         void* d_tokens, int64_t rows, int64_t seqlen, int dtype, void* workspace,
                         size_t workspace_bytes, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, nullptr, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_forward_from(const void* gates, const void* tokens, const void* initial, void* out, int64_t rows,
                       int64_t seqlen, int dtype, int reverse, void* workspace, size_t workspace_bytes,
                       void* stream) {
    return forward_checked(gates, tokens, out, initial, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY,
                           Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_from(const void* gates, const void* states, const void* initial, const void* grad_out,
                        void* d_gates, void* d_tokens, void* d_initial, int64_t rows, int64_t seqlen, int dtype,
                        void* workspace, size_t workspace_bytes, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_forward_gated(const void* gate_inputs, const void* tokens, const void* initial, void* out, int64_t rows,
                        int64_t seqlen, int dtype, int gate, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_checked(gate_inputs, tokens, out, initial, rows, seqlen, dtype, 0, gate,
                           Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_gated(const void* gate_inputs, const void* states, const void* initial, const void* grad_out,
                         void* d_gate_inputs, void* d_tokens, void* d_initial, int64_t rows, int64_t seqlen,
                         int dtype, int gate, void* workspace, size_t workspace_bytes, void* stream) {
    return backward_checked(gate_inputs, states, grad_out, d_gate_inputs, d_tokens, initial, d_initial, rows, seqlen,
                            dtype, gate, Workspace{workspace, workspace_bytes}, stream);
}

unsigned int ascan_workspace_timeouts(const void* workspace_header_copy) {
    return static_cast<const SplitHeader*>(workspace_header_copy)->timeouts;
}

const char* ascan_status_string(int status) {
    switch (status) {
        case ASCAN_OK: return "ok";
        case ASCAN_ERR_NULL_POINTER: return "a required buffer pointer is NULL";
        case ASCAN_ERR_BAD_SHAPE: return "rows or seqlen is negative, or rows exceeds the grid limit";
        case ASCAN_ERR_BAD_DTYPE: return "unsupported dtype: expecting float32, bfloat16, float16, complex64 or complex64 with float32 tokens";
        case ASCAN_ERR_MISALIGNED: return "a buffer is not aligned to its element size";
        case ASCAN_ERR_LAUNCH: return "the HIP runtime reported a launch error";
        case ASCAN_ERR_BAD_ACTIVATION:
            return "unsupported gate activation: expecting identity, or sigmoid with float32, bfloat16 or float16";
        default: return "unknown status";
    }
}

int ascan_last_hip_error(void) { return g_last_hip_error; }

int ascan_abi_version(void) { return ASCAN_ABI_VERSION; }

}  // extern "C"
