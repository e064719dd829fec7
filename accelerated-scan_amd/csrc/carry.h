// Carries between the waves of a row and between the tiles of a row, for
// workgroups that own whole rows.

#ifndef ASCAN_CARRY_H_
#define ASCAN_CARRY_H_

#include "values.h"

namespace ascan {
namespace {

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
// RESET: a total with a gate product of exactly zero discards the incoming state
// (see carry_in).
// With W > 1 the W waves of a row exchange their sub-tile totals through
// `slots`, the row's W entries of one of two buffers selected by `parity`.
template <class V, int W, int U, bool RESET>
__device__ __forceinline__ void exchange_carries(const V (&totA)[U], const V (&totX)[U], V& carry, V& c,
                                                 V* slots, int parity, int w, int lane) {
    if constexpr (W == 1) {
        c = carry;
        V n = carry;
#pragma unroll
        for (int j = 0; j < U; ++j) n = carry_in<RESET>(totA[j], n, totX[j]);
        carry = n;
    } else {
        V TA = totA[0], TX = totX[0];
#pragma unroll
        for (int j = 1; j < U; ++j) {
            TX = carry_in<RESET>(totA[j], TX, totX[j]);
            TA = gate_product<RESET>(TA, totA[j]);
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
            run = carry_in<RESET>(Ai, run, Xi);
        }
        c = mine;
        carry = run;
    }
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_CARRY_H_
