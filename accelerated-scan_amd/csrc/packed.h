// Short rows scanned in groups: cuts between the rows of a group.

#ifndef ASCAN_PACKED_H_
#define ASCAN_PACKED_H_

#include "traits.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Packed rows: short rows, many of them.  One workgroup per row would leave
// most lanes idle (a row of 16 elements occupies 4 lanes of one wave), so a
// workgroup scans a group of consecutive rows -- one contiguous stretch of
// memory -- as a single long row with a "cut" in front of every row: at a row's
// first element the gate is replaced by 0, which annihilates whatever the scan
// carries in from the row before (the scan's combine steps treat a gate of
// exactly zero as a reset, so that even a non-finite state stops at the cut),
// and gate * x[-1] is added to the token.  All
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
//
// Rows at least as long as a vector put at most one such element into a
// vector: it is located once per vector (locate_cut; the kernel keeps the answer
// for its second pass over the registers) and the elements only compare their
// compile-time index with it.  Shorter rows take the element-by-element walk
// every time.
template <class V>
struct CutAt {
    int at;   // index of the element in the vector, or -1
    V start;  // the state its row starts from
};

template <class Tr, bool REV>
__device__ __forceinline__ CutAt<typename Tr::V> locate_cut(int rel0, const Cuts<Tr>& cuts) {
    using V = typename Tr::V;
    CutAt<V> found{-1, vzero<V>()};
    if (cuts.T >= Tr::EPV) {  // wave-uniform
        int row, pos;
        split_position(rel0, cuts.T, cuts.inv_T, row, pos);
        // forward: the row's first element (pos 0); reverse: its last (pos T-1)
        const int at = REV ? cuts.T - 1 - pos : (pos == 0 ? 0 : cuts.T - pos);
        const int cut_row = REV ? row : row + (pos != 0);
        const bool valid = at < Tr::EPV && (unsigned)(rel0 + at) < (unsigned)cuts.len;
        if (valid) found.at = at;
        if (cuts.stage != nullptr && valid) found.start = Tr::load1(cuts.stage + (cut_row - cuts.first_row));
    }
    return found;
}

template <class Tr, bool REV>
__device__ __forceinline__ void cut_rows(typename Tr::V (&g)[Tr::EPV], typename Tr::V (&t)[Tr::EPV], int rel0,
                                         const Cuts<Tr>& cuts, const CutAt<typename Tr::V>& found) {
    using V = typename Tr::V;
    if (cuts.T >= Tr::EPV) {  // wave-uniform
#pragma unroll
        for (int e = 0; e < Tr::EPV; ++e) {
            const bool cut = found.at == e;
            t[e] = vselect(cut, vfma(g[e], found.start, t[e]), t[e]);
            g[e] = vselect(cut, vzero<V>(), g[e]);
        }
        return;
    }
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
// `before[e]` the state that precedes it, both in the order of the scan being
// differentiated (REV = true: forward in time, as the backward kernel names its
// own direction; false: a reverse scan, whose first element is the row's last in
// memory); at a row's last element nothing follows (0), at its first the state
// before it is the row's initial state.  is_first[e] / row_of[e] tell the caller
// where to put the gradient of that initial state.  Rows at least as long as a
// vector have at most one first and one last element in a vector (as above).
template <class Tr, bool REV>
__device__ __forceinline__ void cut_rows_backward(typename Tr::V (&after)[Tr::EPV], typename Tr::V (&before)[Tr::EPV],
                                                  bool (&is_first)[Tr::EPV], int (&row_of)[Tr::EPV], int rel0,
                                                  const Cuts<Tr>& cuts) {
    using V = typename Tr::V;
    int row, pos;
    split_position(rel0, cuts.T, cuts.inv_T, row, pos);
    if (cuts.T >= Tr::EPV) {  // wave-uniform
        // where a row starts (pos 0) and where a row ends (pos T-1) inside this vector, in memory order
        const int low_e = pos == 0 ? 0 : cuts.T - pos;
        const int high_e = cuts.T - 1 - pos;
        const int low_row = row + (pos != 0);
        const int first_e = REV ? low_e : high_e;  // first element of its row in the differentiated scan's order
        const int last_e = REV ? high_e : low_e;
        const int first_row = REV ? low_row : row;
        const bool first_valid = first_e < Tr::EPV && (unsigned)(rel0 + first_e) < (unsigned)cuts.len;
        const bool last_valid = last_e < Tr::EPV && (unsigned)(rel0 + last_e) < (unsigned)cuts.len;
        const int first_at = first_valid ? first_e : -1;
        const int last_at = last_valid ? last_e : -1;
        V start = vzero<V>();
        if (cuts.stage != nullptr && first_valid) start = Tr::load1(cuts.stage + (first_row - cuts.first_row));
#pragma unroll
        for (int e = 0; e < Tr::EPV; ++e) {
            const bool first = first_at == e;
            before[e] = vselect(first, start, before[e]);
            after[e] = vselect(last_at == e, vzero<V>(), after[e]);
            is_first[e] = first;
            row_of[e] = first_row;
        }
        return;
    }
#pragma unroll
    for (int e = 0; e < Tr::EPV; ++e) {
        const bool valid = (unsigned)(rel0 + e) < (unsigned)cuts.len;
        const bool first = valid && pos == (REV ? 0 : cuts.T - 1);
        const bool last = valid && pos == (REV ? cuts.T - 1 : 0);
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

}  // namespace
}  // namespace ascan

#endif  // ASCAN_PACKED_H_
