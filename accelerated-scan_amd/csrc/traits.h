// Storage formats of the scan: how 16-byte vectors of each dtype unpack to
// fp32 (or complex) values and pack back.

#ifndef ASCAN_TRAITS_H_
#define ASCAN_TRAITS_H_

#include "values.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Storage traits: S = element type in memory, V = arithmetic type,
// EPV = elements per 16-byte vector.
// ---------------------------------------------------------------------------
typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));  // one 16-byte vector
typedef unsigned int u32x2_t __attribute__((ext_vector_type(2)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));  // four words of LDS at a time
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

}  // namespace
}  // namespace ascan

#endif  // ASCAN_TRAITS_H_
