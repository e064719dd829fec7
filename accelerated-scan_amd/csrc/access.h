// Global-memory access of the scan kernels: row windows, masked vector loads
// and stores, tile geometry.

#ifndef ASCAN_ACCESS_H_
#define ASCAN_ACCESS_H_

#include "traits.h"

namespace ascan {
namespace {

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

}  // namespace
}  // namespace ascan

#endif  // ASCAN_ACCESS_H_
