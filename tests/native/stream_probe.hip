// Streaming probe for MI355X (gfx950): kernels that move the same bytes as the
// scan kernels, with the same 16-byte nontemporal accesses, and do no
// arithmetic worth the name.  What they reach is what the memory system
// delivers for a given mix of reads and writes and a given order of access;
// bench.py reports it beside the scan's own figure as the device ceiling.
// Measurement infrastructure: nothing in the library depends on it.
//
//   pattern 0  linear sweep: workgroup i moves the i-th 16 KiB of every tensor
//              (consecutive workgroups touch consecutive memory);
//   pattern 1  row walk: one 1024-thread workgroup per row, walking the row in
//              tiles of 64 KiB (16 waves x 4 KiB), as the scan kernels do for
//              long rows, without their barrier;
//   pattern 2  row walk with one workgroup barrier per tile;
//   pattern 3  linear sweep in the row walk's units: workgroup i moves the i-th
//              tile of every tensor (barrier) and ends;
//   pattern 4  row walk by `row_step` persistent workgroups: workgroup b walks
//              rows b, b + row_step, ... (fewer rows in flight than compute units
//              when row_step is below their number).
//   pattern 5  ticket sweep (stream_probe_sweep): persistent 1024-thread workgroups
//              take tiles in memory order from one ticket counter, so that the
//              stretch of memory in flight stays compact however long the rows are;
//   pattern 6  ticket sweep in which a tile may store only after the earlier tiles
//              of its row have announced that their loads have landed -- one
//              64-byte record per tile, lane i of wave 0 reads record n-1-i with
//              device-scope loads -- i.e. with the dependency (and the idle round
//              trip) of a scan whose tiles pass carries through global memory.
// `blocks_per_wave` in {1, 2, 4, 8} sets the tile of patterns 1-3 and 5-6: that many KiB
// per wave, 16 times as much per workgroup (the scan kernels: 4, 64 KiB tiles).
// `row_step` > 1 (patterns 1, 2) hands consecutive workgroups rows that far apart.
// `lds_bytes` of dynamic LDS are requested per workgroup (nothing uses them):
// more than half a compute unit's LDS keeps workgroups from sharing one.
//
// `reads` of the three inputs are read and `writes` of the two outputs are
// written; every tensor is rows x row_bytes bytes, dense.

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

constexpr int kThreads = 1024;
constexpr int64_t kChunk = (int64_t)kThreads * 16;  // bytes one workgroup moves per tensor in one go
// row walk: a wave moves BPW KiB of every tensor per tile (the scan kernels: 4)
constexpr int64_t tile_bytes(int bpw) { return (int64_t)kThreads * 16 * bpw; }

struct Tensors {
    const u32x4_t* in[3];
    u32x4_t* out[2];
};

// Read-only probes: a store that the data never triggers keeps the loads alive.
__device__ __forceinline__ void keep(u32x4_t s, u32x4_t* where) {
    if ((s.x ^ s.y ^ s.z ^ s.w) == 0x9e3779b9u && s.x == 0x7f4a7c15u) *where = s;
}

template <int NR, int NW>
__global__ void __launch_bounds__(kThreads) stream_probe_linear(Tensors t) {
    const int64_t v = (int64_t)blockIdx.x * kThreads + threadIdx.x;  // vector index
    u32x4_t s = {1u, 2u, 3u, 4u};
#pragma unroll
    for (int r = 0; r < NR; ++r) s += __builtin_nontemporal_load(t.in[r] + v);
#pragma unroll
    for (int w = 0; w < NW; ++w) __builtin_nontemporal_store(s + (unsigned)w, t.out[w] + v);
    if constexpr (NW == 0) keep(s, t.out[0] + v);
}

template <int NR, int NW, bool BARRIER, int BPW>
__global__ void __launch_bounds__(kThreads) stream_probe_rows(Tensors t, int64_t row_vectors, int row_step, int64_t rows) {
    constexpr int kBlocksPerWave = BPW;
    constexpr int64_t kTile = tile_bytes(BPW);
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    // one row per workgroup; with row_vectors == one tile, the launch is a linear sweep in tiles.
    // row_step > 1: consecutive workgroups take rows row_step apart (all rows are still covered).
    // rows > gridDim.x (pattern 4): the workgroups are persistent and take rows b, b + gridDim.x, ...
    for (int64_t first = blockIdx.x; first < rows; first += gridDim.x) {
    const int64_t per_pass = rows / row_step;
    const int64_t row_index = row_step > 1 ? (first % per_pass) * row_step + first / per_pass : first;
    const int64_t row = row_index * row_vectors;
    for (int64_t tile = 0; tile < row_vectors; tile += kTile / 16) {
        const int64_t base = row + tile + (int64_t)wave * (64 * kBlocksPerWave) + lane;
        u32x4_t s[kBlocksPerWave];
#pragma unroll
        for (int j = 0; j < kBlocksPerWave; ++j) {
            s[j] = u32x4_t{1u, 2u, 3u, 4u};
#pragma unroll
            for (int r = 0; r < NR; ++r) s[j] += __builtin_nontemporal_load(t.in[r] + base + j * 64);
        }
        if constexpr (BARRIER) __syncthreads();
#pragma unroll
        for (int j = 0; j < kBlocksPerWave; ++j) {
#pragma unroll
            for (int w = 0; w < NW; ++w) __builtin_nontemporal_store(s[j] + (unsigned)w, t.out[w] + base + j * 64);
            if constexpr (NW == 0) keep(s[j], t.out[0] + base + j * 64);
        }
    }
    }
}

// Patterns 5 and 6.  table: [0] the ticket counter, then one 64-byte record per tile from
// byte 64 on; cleared by the caller before every launch.  Every wait is bounded; waits that
// ran out are counted in table word 1.
template <int NR, int NW, bool CHAIN, int BPW>
__global__ void __launch_bounds__(kThreads) stream_probe_tickets(Tensors t, int64_t total_tiles, int tiles_per_row,
                                                                unsigned long long* table) {
    __shared__ long long mailbox;
    __shared__ unsigned int carry_word;
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    constexpr int64_t kTileVec = tile_bytes(BPW) / 16;
    unsigned long long* flags = table + 8;
    for (;;) {
        if (threadIdx.x == 0) {
            const long long n = (long long)__hip_atomic_fetch_add(table, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            mailbox = n < total_tiles ? n : -1;
        }
        __syncthreads();
        const long long tile = __builtin_amdgcn_readfirstlane((int)mailbox);
        __syncthreads();
        if (tile < 0) break;
        const int64_t base = tile * kTileVec + (int64_t)wave * (64 * BPW) + lane;
        u32x4_t s[BPW];
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
            s[j] = u32x4_t{1u, 2u, 3u, 4u};
#pragma unroll
            for (int r = 0; r < NR; ++r) s[j] += __builtin_nontemporal_load(t.in[r] + base + j * 64);
        }
        unsigned int c = 0;
        if constexpr (CHAIN) {
            __syncthreads();  // everybody's loads have landed (the sums above consumed them)
            if (wave == 0) {
                if (lane == 0) {
                    __hip_atomic_store(flags + tile * 8, (unsigned long long)(tile + 1), __ATOMIC_RELAXED,
                                       __HIP_MEMORY_SCOPE_AGENT);
                }
                const int k = (int)(tile % tiles_per_row);
                unsigned int got = 0;
                if (lane < k) {
                    const unsigned long long want = (unsigned long long)(tile - lane);  // record tile-1-lane holds tile-lane
                    for (unsigned spins = 0;; ++spins) {
                        const unsigned long long v = __hip_atomic_load(flags + (tile - 1 - lane) * 8, __ATOMIC_RELAXED,
                                                                       __HIP_MEMORY_SCOPE_AGENT);
                        if (v == want) {
                            got = (unsigned int)v;
                            break;
                        }
                        if (spins > 4000000u) {
                            atomicAdd(reinterpret_cast<unsigned int*>(table + 1), 1u);
                            break;
                        }
                        __builtin_amdgcn_s_sleep(1);
                    }
                }
                for (int o = 32; o > 0; o >>= 1) got += __shfl_xor(got, o);
                if (lane == 0) carry_word = got;
            }
            __syncthreads();
            c = carry_word;
        }
#pragma unroll
        for (int j = 0; j < BPW; ++j) {
#pragma unroll
            for (int w = 0; w < NW; ++w) __builtin_nontemporal_store(s[j] + (unsigned)w + c, t.out[w] + base + j * 64);
            if constexpr (NW == 0) keep(s[j], t.out[0] + base + j * 64);
        }
    }
}

template <class K>
hipError_t allow_lds(K kernel, unsigned lds_bytes) {
    if (lds_bytes <= 64u * 1024u) return hipSuccess;
    return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                               (int)lds_bytes);
}

template <int NR, int NW, int BPW>
hipError_t launch_rows(const Tensors& t, int64_t rows, int64_t row_bytes, int pattern, int row_step,
                       unsigned lds_bytes, hipStream_t stream) {
    hipError_t e = pattern == 1 ? allow_lds(stream_probe_rows<NR, NW, false, BPW>, lds_bytes)
                                : allow_lds(stream_probe_rows<NR, NW, true, BPW>, lds_bytes);
    if (e != hipSuccess) return e;
    if (pattern == 1) {
        hipLaunchKernelGGL((stream_probe_rows<NR, NW, false, BPW>), dim3((unsigned)rows), dim3(kThreads), lds_bytes,
                           stream, t, row_bytes / 16, row_step, rows);
    } else if (pattern == 2) {
        hipLaunchKernelGGL((stream_probe_rows<NR, NW, true, BPW>), dim3((unsigned)rows), dim3(kThreads), lds_bytes,
                           stream, t, row_bytes / 16, row_step, rows);
    } else if (pattern == 4) {  // row_step is the number of persistent workgroups
        hipLaunchKernelGGL((stream_probe_rows<NR, NW, true, BPW>), dim3((unsigned)row_step), dim3(kThreads), lds_bytes,
                           stream, t, row_bytes / 16, 1, rows);
    } else {
        const int64_t tiles = rows * row_bytes / tile_bytes(BPW);
        hipLaunchKernelGGL((stream_probe_rows<NR, NW, true, BPW>), dim3((unsigned)tiles), dim3(kThreads), lds_bytes,
                           stream, t, tile_bytes(BPW) / 16, 1, tiles);
    }
    return hipGetLastError();
}

template <int NR, int NW>
hipError_t launch(const Tensors& t, int64_t rows, int64_t row_bytes, int pattern, int bpw, int row_step,
                  unsigned lds_bytes, hipStream_t stream) {
    if (pattern == 0) {
        const hipError_t e = allow_lds(stream_probe_linear<NR, NW>, lds_bytes);
        if (e != hipSuccess) return e;
        const int64_t blocks = rows * row_bytes / kChunk;
        hipLaunchKernelGGL((stream_probe_linear<NR, NW>), dim3((unsigned)blocks), dim3(kThreads), lds_bytes, stream, t);
        return hipGetLastError();
    }
    switch (bpw) {
        case 1: return launch_rows<NR, NW, 1>(t, rows, row_bytes, pattern, row_step, lds_bytes, stream);
        case 2: return launch_rows<NR, NW, 2>(t, rows, row_bytes, pattern, row_step, lds_bytes, stream);
        case 8: return launch_rows<NR, NW, 8>(t, rows, row_bytes, pattern, row_step, lds_bytes, stream);
        default: return launch_rows<NR, NW, 4>(t, rows, row_bytes, pattern, row_step, lds_bytes, stream);
    }
}

template <int NR, int NW>
hipError_t launch_tickets(const Tensors& t, int64_t total_tiles, int tiles_per_row, bool chain, int bpw,
                          unsigned long long* table, unsigned grid, hipStream_t stream) {
    auto go = [&](auto kernel) {
        hipLaunchKernelGGL(kernel, dim3(grid), dim3(kThreads), 0, stream, t, total_tiles, tiles_per_row, table);
        return hipGetLastError();
    };
    if (bpw == 2) return chain ? go(stream_probe_tickets<NR, NW, true, 2>) : go(stream_probe_tickets<NR, NW, false, 2>);
    return chain ? go(stream_probe_tickets<NR, NW, true, 4>) : go(stream_probe_tickets<NR, NW, false, 4>);
}

}  // namespace

// Patterns 5 (chain = 0) and 6 (chain = 1): `grid` persistent workgroups sweep rows x row_bytes
// bytes of every tensor in tiles of 16 * blocks_per_wave KiB (blocks_per_wave in {2, 4}).  `table`
// holds 64 bytes plus 64 bytes per tile and must be zero when the launch starts.  Returns 0, -1
// for arguments the kernels do not cover, or a hipError_t.
extern "C" __attribute__((visibility("default"))) int stream_probe_sweep(
    const void* in0, const void* in1, const void* in2, void* out0, void* out1, int64_t rows, int64_t row_bytes,
    int reads, int writes, int chain, int blocks_per_wave, void* table, size_t table_bytes, unsigned grid,
    void* stream) {
    if (rows <= 0 || row_bytes <= 0 || grid == 0 || (blocks_per_wave != 2 && blocks_per_wave != 4)) return -1;
    const int64_t tile = tile_bytes(blocks_per_wave);
    if (row_bytes % tile != 0 || row_bytes / tile > 64) return -1;
    const int64_t total_tiles = rows * (row_bytes / tile);
    if (total_tiles > 2147483647LL || !table || reinterpret_cast<uintptr_t>(table) % 64 ||
        table_bytes < 64 + (size_t)total_tiles * 64) {
        return -1;
    }
    const void* ins[3] = {in0, in1, in2};
    void* outs[2] = {out0, out1};
    for (int r = 0; r < reads; ++r)
        if (r >= 3 || !ins[r] || reinterpret_cast<uintptr_t>(ins[r]) % 16) return -1;
    for (int w = 0; w < (writes > 0 ? writes : 1); ++w)
        if (w >= 2 || !outs[w] || reinterpret_cast<uintptr_t>(outs[w]) % 16) return -1;
    Tensors t;
    for (int r = 0; r < 3; ++r) t.in[r] = static_cast<const u32x4_t*>(ins[r]);
    for (int w = 0; w < 2; ++w) t.out[w] = static_cast<u32x4_t*>(outs[w]);
    hipStream_t s = static_cast<hipStream_t>(stream);
    auto* words = static_cast<unsigned long long*>(table);
    const int per_row = (int)(row_bytes / tile);
    switch (reads * 10 + writes) {
        case 32: return (int)launch_tickets<3, 2>(t, total_tiles, per_row, chain != 0, blocks_per_wave, words, grid, s);
        case 21: return (int)launch_tickets<2, 1>(t, total_tiles, per_row, chain != 0, blocks_per_wave, words, grid, s);
        default: return -1;
    }
}

// Returns 0, -1 for arguments the kernels do not cover, or a hipError_t.
extern "C" __attribute__((visibility("default"))) int stream_probe_launch(
    const void* in0, const void* in1, const void* in2, void* out0, void* out1, int64_t rows, int64_t row_bytes,
    int reads, int writes, int pattern, int blocks_per_wave, int row_step, unsigned lds_bytes, void* stream) {
    if (row_step < 1 || (pattern != 4 && rows % row_step != 0)) return -1;
    if (rows <= 0 || row_bytes <= 0 || pattern < 0 || pattern > 4 || lds_bytes > 160u * 1024u) return -1;
    if (blocks_per_wave != 1 && blocks_per_wave != 2 && blocks_per_wave != 4 && blocks_per_wave != 8) return -1;
    if (pattern == 0 ? (rows * row_bytes) % kChunk != 0 : row_bytes % tile_bytes(blocks_per_wave) != 0) return -1;
    if (rows * row_bytes / kChunk > 2147483647LL || rows > 2147483647LL) return -1;
    const void* ins[3] = {in0, in1, in2};
    void* outs[2] = {out0, out1};
    for (int r = 0; r < reads; ++r)
        if (r >= 3 || !ins[r] || reinterpret_cast<uintptr_t>(ins[r]) % 16) return -1;
    for (int w = 0; w < (writes > 0 ? writes : 1); ++w)  // read-only probes still name out0 (never written)
        if (w >= 2 || !outs[w] || reinterpret_cast<uintptr_t>(outs[w]) % 16) return -1;
    Tensors t;
    for (int r = 0; r < 3; ++r) t.in[r] = static_cast<const u32x4_t*>(ins[r]);
    for (int w = 0; w < 2; ++w) t.out[w] = static_cast<u32x4_t*>(outs[w]);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const int mix = reads * 10 + writes;
    switch (mix) {
        case 32: return (int)launch<3, 2>(t, rows, row_bytes, pattern, blocks_per_wave, row_step, lds_bytes, s);
        case 21: return (int)launch<2, 1>(t, rows, row_bytes, pattern, blocks_per_wave, row_step, lds_bytes, s);
        case 11: return (int)launch<1, 1>(t, rows, row_bytes, pattern, blocks_per_wave, row_step, lds_bytes, s);
        case 30: return (int)launch<3, 0>(t, rows, row_bytes, pattern, blocks_per_wave, row_step, lds_bytes, s);
        case 2: return (int)launch<0, 2>(t, rows, row_bytes, pattern, blocks_per_wave, row_step, lds_bytes, s);
        default: return -1;
    }
}
