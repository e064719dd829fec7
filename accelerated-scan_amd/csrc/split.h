// Rows split over many workgroups: the table in global memory, the hand-out
// of tiles by ticket and the decoupled look-back.

#ifndef ASCAN_SPLIT_H_
#define ASCAN_SPLIT_H_

#include "carry.h"

namespace ascan {
namespace {

// ---------------------------------------------------------------------------
// Split rows: several workgroups per row, for calls with too few rows to
// occupy the machine.  A workgroup works on one tile of one row at a time; the
// state entering the tile comes from the workgroups of the earlier tiles
// through a small table in global memory (single pass, "decoupled look-back"):
//   * a workgroup publishes its tile's aggregate (A, X) as soon as it has it;
//   * it then walks back over the earlier tiles of its row, folding aggregates
//     until it meets a tile whose inclusive state P is already published;
//   * it publishes its own inclusive state and finishes the tile.
// Tiles are handed out by ticket: every row has a counter, and a workgroup
// takes the next tile of the row it serves with one fetch-add on it.  A tile
// is therefore only ever waited for by workgroups that started after its
// owner did: progress never depends on a workgroup that has not been
// dispatched yet, whatever else is running on the GPU, and the launch size
// (what an idle GPU holds at once) is a matter of speed only.  One counter per
// row keeps the fetch-adds of different rows apart (measured: ~11 ns each on
// one address on an idle GPU, ~60 ns under streaming load; concurrent across
// addresses).  Each wait is nevertheless bounded by a limit set by the host;
// a wait that runs out poisons the result with NaN and is counted in the
// header.  Waiting time is summed from clock differences capped at 10 us
// each, so a stretch during which the whole kernel was not running does not
// count.
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
    // the limit occupies words 2 and 3 of the header; every word has exactly one writer
    if (i < nwords) words[i] = i == 2 ? (uint32_t)wait_limit : (i == 3 ? (uint32_t)(wait_limit >> 32) : 0u);
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

// Hands the workgroup its next tile.  Workgroup b serves row b % rows -- with
// fewer rows than workgroups several workgroups share a row and draw its tiles
// in turn -- and, when that row has no tiles left, the rows b + G, b + 2G, ...
// (G = workgroups in the launch), so every row is served whatever G is.
// (Letting idle workgroups look for tiles in other rows was tried: near the end
// hundreds of them draw from the few counters that still have tiles, and the
// owners' own draws queue behind them.)  Returns false when the workgroup has
// nothing left to do.  All threads of the workgroup call it together and get
// the same answer; `mailbox` is two words of LDS.
__device__ __forceinline__ bool take_split_tile(SplitHeader* header, int64_t rows, int64_t ntiles, SplitWalk& walk,
                                                int64_t& row, int64_t& k, long long* mailbox) {
    if (threadIdx.x < 64) {  // wave 0
        const int lane = threadIdx.x;
        SplitTicket* tickets = split_tickets(header);
        long long got_row = -1, got_k = -1;
        while (walk.row < rows) {
            const unsigned long long ticket =
                from_lane0(walk.has_drawn ? walk.drawn : draw_ticket(&tickets[walk.row], lane));
            walk.has_drawn = false;
            if (ticket < (unsigned long long)ntiles) {
                got_row = walk.row;
                got_k = (long long)ticket;
                if (ticket + 1 < (unsigned long long)ntiles) {  // draw the next one now; it is read at the next call
                    walk.drawn = draw_ticket(&tickets[walk.row], lane);
                    walk.has_drawn = true;
                }
                break;
            }
            walk.row += gridDim.x;  // this row is handed out completely
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
//
// Wave 0 walks back over the row's earlier tiles while it holds its sub-tile in
// registers like every other wave, and the walk needs registers of its own.
// `set_aside()` / `take_back()` are called by wave 0 only, around the walk: the
// kernels park their raw vectors in LDS there, which frees those registers for
// the walk without a trip through scratch memory.
template <class V, int W, int U, class SetAside, class TakeBack>
__device__ __forceinline__ void exchange_carries_split(const V (&totA)[U], const V (&totX)[U], V& c, V* slots,
                                                       int w, int lane, SplitHeader* header, SplitRecord* mine,
                                                       int64_t stride, int64_t k, V row_start, SetAside set_aside,
                                                       TakeBack take_back) {
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
        set_aside();
        const V carry_in = split_look_back(header, mine, stride, k, runA, runX, row_start, lane);
        if (lane == 0) *carry_slot = carry_in;
        take_back();
    }
    __syncthreads();
    c = vfma(mineA, *carry_slot, mineX);
}

}  // namespace
}  // namespace ascan

#endif  // ASCAN_SPLIT_H_
