// Hop probe for MI355X (gfx950): what it costs one workgroup to hand a word to another
// through global memory, which is what a scan pays when the tiles of a row are spread
// over workgroups.  Measurement infrastructure: nothing in the library depends on it.
//
//   hop        a publish -> peek ping-pong between two single-wave workgroups, 64-bit words
//              on cache lines of their own.  Pairs are placed on the same XCD and on
//              different XCDs (workgroups are dealt to the XCDs round robin; every workgroup
//              reads its XCC id from the hardware register and the pairs are classified by
//              what they read).  Two flavours of access: device scope (sc1: what the
//              split-row table of the library uses), and workgroup scope (sc0), which the
//              other compute unit never sees -- a load of that scope may be served by the
//              reader's own vector cache -- so the pairs run into their (bounded) wait limit;
//   fetch-add  a dependent chain of device-scope fetch-adds, every workgroup on a counter of
//              its own or all on one.
// Each is measured on an idle GPU and while a second stream runs the row-walk kernel of the
// streaming probe (one 1024-thread workgroup per 256 KiB row, 3 reads + 2 writes) over
// 12288 rows, i.e. under the load the scan kernels themselves put on the memory system.
//
// usage: hop_probe [rows] [row_bytes]     (defaults 12288 262144)
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>
#include <vector>

#define CHECK(x)                                                                              \
    do {                                                                                      \
        hipError_t e_ = (x);                                                                  \
        if (e_ != hipSuccess) {                                                               \
            printf("HIP error %s at %s:%d\n", hipGetErrorString(e_), __FILE__, __LINE__);     \
            fflush(stdout);                                                                   \
            exit(1);                                                                          \
        }                                                                                     \
    } while (0)

typedef unsigned int u32x4_t __attribute__((ext_vector_type(4)));

// XCC_ID, bits [3:0] of hardware register 20
__device__ __forceinline__ int xcc_id() { return (int)__builtin_amdgcn_s_getreg((3 << 11) | 20) & 0xf; }

template <bool DEVICE_SCOPE>
__device__ __forceinline__ void put(unsigned long long* p, unsigned long long v) {
    if constexpr (DEVICE_SCOPE) {
        __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        asm volatile("global_store_dwordx2 %0, %1, off sc0" ::"v"(p), "v"(v) : "memory");
    }
}
template <bool DEVICE_SCOPE>
__device__ __forceinline__ unsigned long long get(unsigned long long* p) {
    if constexpr (DEVICE_SCOPE) {
        return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
        unsigned long long v;
        asm volatile("global_load_dwordx2 %0, %1, off sc0\n\ts_waitcnt vmcnt(0)" : "=v"(v) : "v"(p) : "memory");
        return v;
    }
}

// Workgroup b plays role[b] (0 serves, 1 returns) in pair partner[b] (-1: none).  Every wait is
// bounded by spin_limit looks; a pair that runs out stops and is reported in fails[pair].
template <bool DEVICE_SCOPE>
__global__ void pingpong(unsigned long long* lines, const int* partner, const int* role, int rounds,
                         unsigned long long* ticks, int* xcc, int* fails, unsigned long long spin_limit) {
    const int b = blockIdx.x;
    if (threadIdx.x != 0) return;
    xcc[b] = xcc_id();
    const int pair = partner[b];
    if (pair < 0) return;
    unsigned long long* there = lines + (size_t)pair * 32;      // pairs 256 bytes apart
    unsigned long long* back = lines + (size_t)pair * 32 + 16;  // the answer 128 bytes further
    const bool serves = role[b] == 0;
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    int failed = 0;
    for (int r = 1; r <= rounds && !failed; ++r) {
        if (serves) put<DEVICE_SCOPE>(there, (unsigned long long)r);
        unsigned long long looks = 0;
        while (get<DEVICE_SCOPE>(serves ? back : there) != (unsigned long long)r) {
            if (++looks > spin_limit) {
                failed = 1;
                break;
            }
        }
        if (!serves && !failed) put<DEVICE_SCOPE>(back, (unsigned long long)r);
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();  // 100 MHz
    if (serves) ticks[pair] = t1 - t0;
    if (failed) fails[pair] = 1;
}

__global__ void fetch_adds(unsigned long long* counters, int shared, int n, unsigned long long* ticks) {
    if (threadIdx.x != 0) return;
    unsigned long long* c = counters + (shared ? 0 : (size_t)blockIdx.x * 32);
    const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
    unsigned long long acc = 0;
    for (int i = 0; i < n; ++i) {
        acc += __hip_atomic_fetch_add(c, 1ull, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        c += (acc >> 63);  // the next address depends on the result (always + 0)
    }
    const unsigned long long t1 = __builtin_amdgcn_s_memrealtime();
    ticks[blockIdx.x] = t1 - t0 + (acc >> 63);
}

struct Tensors {
    const u32x4_t* in[3];
    u32x4_t* out[2];
};

// the load: one 1024-thread workgroup per row, 64 KiB tiles, a barrier per tile
__global__ void __launch_bounds__(1024) row_walk(Tensors t, int64_t row_vectors) {
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    const int64_t row = (int64_t)blockIdx.x * row_vectors;
    for (int64_t tile = 0; tile < row_vectors; tile += 4096) {
        const int64_t base = row + tile + wave * 256 + lane;
        u32x4_t s[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            s[j] = u32x4_t{1u, 2u, 3u, 4u};
#pragma unroll
            for (int r = 0; r < 3; ++r) s[j] += __builtin_nontemporal_load(t.in[r] + base + j * 64);
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int w = 0; w < 2; ++w) __builtin_nontemporal_store(s[j] + (unsigned)w, t.out[w] + base + j * 64);
    }
}

struct Setup {
    Tensors t;
    int64_t rows, row_bytes;
    hipStream_t probe_stream, load_stream;
};

static void start_load(const Setup& s) {
    for (int i = 0; i < 4; ++i)
        hipLaunchKernelGGL(row_walk, dim3((unsigned)s.rows), dim3(1024), 0, s.load_stream, s.t, s.row_bytes / 16);
}

static void print_stats(const char* label, std::vector<double>& v, int timeouts) {
    if (v.empty()) {
        printf("  %-10s none completed (%d pairs ran into the wait limit)\n", label, timeouts);
        return;
    }
    std::sort(v.begin(), v.end());
    printf("  %-10s %2zu pairs: min %5.0f  median %5.0f  max %5.0f ns per hop (%d ran into the wait limit)\n", label, v.size(),
           v.front(), v[v.size() / 2], v.back(), timeouts);
}

template <bool DEVICE_SCOPE>
static void run_hops(const Setup& s, bool loaded) {
    // 64 workgroups, 32 pairs: (b, b + 8) lands on one XCD when workgroups are dealt round robin,
    // (b, b + 1) on two; the pairs are classified by the XCC ids the workgroups report
    const int nblocks = 64;
    std::vector<int> partner(nblocks, -1), role(nblocks, 0), first, second;
    auto pair_up = [&](int a, int b) {
        partner[a] = partner[b] = (int)first.size();
        role[b] = 1;
        first.push_back(a);
        second.push_back(b);
    };
    for (int base : {0, 32})
        for (int i = 0; i < 8; ++i) pair_up(base + i, base + i + 8);
    for (int base : {16, 48})
        for (int i = 0; i < 16; i += 2) pair_up(base + i, base + i + 1);
    const int npairs = (int)first.size();
    const int rounds = loaded ? 2000 : 5000;
    int *d_partner, *d_role, *d_xcc, *d_fails;
    unsigned long long *lines, *d_ticks;
    CHECK(hipMalloc(&d_partner, nblocks * 4));
    CHECK(hipMalloc(&d_role, nblocks * 4));
    CHECK(hipMalloc(&d_xcc, nblocks * 4));
    CHECK(hipMalloc(&d_fails, npairs * 4));
    CHECK(hipMalloc(&lines, (size_t)npairs * 256));
    CHECK(hipMalloc(&d_ticks, npairs * 8));
    CHECK(hipMemcpy(d_partner, partner.data(), nblocks * 4, hipMemcpyHostToDevice));
    CHECK(hipMemcpy(d_role, role.data(), nblocks * 4, hipMemcpyHostToDevice));
    CHECK(hipMemset(d_fails, 0, npairs * 4));
    CHECK(hipMemset(d_ticks, 0, npairs * 8));
    CHECK(hipMemset(lines, 0, (size_t)npairs * 256));
    CHECK(hipDeviceSynchronize());
    hipLaunchKernelGGL(pingpong<DEVICE_SCOPE>, dim3(nblocks), dim3(64), 0, s.probe_stream, lines, d_partner, d_role, rounds,
                       d_ticks, d_xcc, d_fails, 2000000ull);
    if (loaded) start_load(s);
    CHECK(hipDeviceSynchronize());
    std::vector<unsigned long long> ticks(npairs);
    std::vector<int> xcc(nblocks), fails(npairs);
    CHECK(hipMemcpy(ticks.data(), d_ticks, npairs * 8, hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(xcc.data(), d_xcc, nblocks * 4, hipMemcpyDeviceToHost));
    CHECK(hipMemcpy(fails.data(), d_fails, npairs * 4, hipMemcpyDeviceToHost));
    std::vector<double> same, other;
    int same_out = 0, other_out = 0;
    for (int p = 0; p < npairs; ++p) {
        const bool one_xcd = xcc[first[p]] == xcc[second[p]];
        if (fails[p]) {
            ++(one_xcd ? same_out : other_out);
        } else {
            (one_xcd ? same : other).push_back((double)ticks[p] * 10.0 / (2.0 * rounds));
        }
    }
    printf("hop, %s, %s:\n", DEVICE_SCOPE ? "device scope (sc1)" : "workgroup scope (sc0)", loaded ? "under load" : "idle GPU");
    print_stats("same XCD", same, same_out);
    print_stats("other XCD", other, other_out);
    fflush(stdout);
    for (void* p : {(void*)d_partner, (void*)d_role, (void*)d_xcc, (void*)d_fails, (void*)lines, (void*)d_ticks}) CHECK(hipFree(p));
}

static void run_fetch_adds(const Setup& s, bool loaded, int shared) {
    const int blocks = 64, n = loaded ? 2000 : 5000;
    unsigned long long *counters, *d_ticks;
    CHECK(hipMalloc(&counters, (size_t)blocks * 256));
    CHECK(hipMalloc(&d_ticks, blocks * 8));
    CHECK(hipMemset(counters, 0, (size_t)blocks * 256));
    CHECK(hipDeviceSynchronize());
    hipLaunchKernelGGL(fetch_adds, dim3(blocks), dim3(64), 0, s.probe_stream, counters, shared, n, d_ticks);
    if (loaded) start_load(s);
    CHECK(hipDeviceSynchronize());
    std::vector<unsigned long long> ticks(blocks);
    CHECK(hipMemcpy(ticks.data(), d_ticks, blocks * 8, hipMemcpyDeviceToHost));
    std::vector<double> v;
    for (int i = 0; i < blocks; ++i) v.push_back((double)ticks[i] * 10.0 / n);
    std::sort(v.begin(), v.end());
    printf("fetch-add, device scope, %s, %d workgroups on %s: min %5.0f  median %5.0f  max %5.0f ns per draw\n",
           loaded ? "under load" : "idle GPU", blocks, shared ? "one counter" : "counters of their own", v.front(),
           v[v.size() / 2], v.back());
    fflush(stdout);
    CHECK(hipFree(counters));
    CHECK(hipFree(d_ticks));
}

int main(int argc, char** argv) {
    Setup s;
    s.rows = argc > 1 ? atoll(argv[1]) : 12288;
    s.row_bytes = argc > 2 ? atoll(argv[2]) : 262144;
    if (s.rows <= 0 || s.row_bytes <= 0 || s.row_bytes % 65536 != 0) {
        printf("usage: hop_probe [rows] [row_bytes: a multiple of 65536]\n");
        return 2;
    }
    const size_t bytes = (size_t)s.rows * s.row_bytes;
    void* bufs[5];
    for (int i = 0; i < 5; ++i) {
        CHECK(hipMalloc(&bufs[i], bytes));
        CHECK(hipMemset(bufs[i], i + 1, bytes));
    }
    for (int i = 0; i < 3; ++i) s.t.in[i] = (const u32x4_t*)bufs[i];
    for (int i = 0; i < 2; ++i) s.t.out[i] = (u32x4_t*)bufs[3 + i];
    CHECK(hipStreamCreate(&s.probe_stream));
    CHECK(hipStreamCreate(&s.load_stream));
    CHECK(hipDeviceSynchronize());
    printf("load: row walk over %lld rows of %lld bytes, 3 reads + 2 writes\n", (long long)s.rows, (long long)s.row_bytes);
    for (int loaded = 0; loaded < 2; ++loaded) {
        run_hops<true>(s, loaded != 0);
        run_hops<false>(s, loaded != 0);
    }
    for (int loaded = 0; loaded < 2; ++loaded) {
        run_fetch_adds(s, loaded != 0, 0);
        run_fetch_adds(s, loaded != 0, 1);
    }
    printf("done\n");
    return 0;
}
