// First-order linear recurrence (scan) for gfx950 (MI355X): the C ABI declared
// in include/ascan.h.  The kernels live in the headers of this directory and
// are compiled per dtype (forward_<dtype>.hip, backward_<dtype>.hip).
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

#include <atomic>

#include "ascan.h"
#include "dispatch.h"
#include "policy.h"

namespace ascan {

thread_local int g_last_hip_error = 0;

namespace {

// Split-row table of ascan_forward_split_static: device memory that belongs to the
// library's code object, so the entry point needs no allocation.  Each GPU the
// library runs on holds its own copy at its own address until the process ends;
// the name below is only a host-side handle for hipGetSymbolAddress, never a
// device address.
static __device__ __align__(256) unsigned char scratch[ASCAN_STATIC_WORKSPACE_BYTES];

// Address of `scratch` on the current device (looked up once per device), or
// null with g_last_hip_error set.
void* static_workspace() {
    constexpr int kMaxDevices = 64;
    static std::atomic<void*> known[kMaxDevices];
    int device = 0;
    hipError_t e = hipGetDevice(&device);
    if (e == hipSuccess && (device < 0 || device >= kMaxDevices)) e = hipErrorInvalidDevice;
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return nullptr;
    }
    void* ptr = known[device].load(std::memory_order_acquire);
    if (ptr == nullptr) {
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess || ptr == nullptr) {
            g_last_hip_error = (int)(e != hipSuccess ? e : hipErrorInvalidSymbol);
            return nullptr;
        }
        known[device].store(ptr, std::memory_order_release);
    }
    return ptr;
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

// A buffer of a call as a byte range (null buffers are empty ranges).
struct Span {
    uintptr_t begin, end;
};
Span span_of(const void* p, int64_t elements, size_t element_bytes) {
    const uintptr_t b = reinterpret_cast<uintptr_t>(p);
    return Span{b, p ? b + (uintptr_t)elements * element_bytes : b};
}
bool overlap(const Span& a, const Span& b) { return a.begin < b.end && b.begin < a.end; }

// True when an output range meets an input range or another output range.
template <size_t NI, size_t NO>
bool outputs_overlap(const Span (&inputs)[NI], const Span (&outputs)[NO]) {
    for (size_t o = 0; o < NO; ++o) {
        for (size_t i = 0; i < NI; ++i)
            if (overlap(outputs[o], inputs[i])) return true;
        for (size_t q = o + 1; q < NO; ++q)
            if (overlap(outputs[o], outputs[q])) return true;
    }
    return false;
}

// Largest row count one launch can address: gridDim.x is limited to 2^31-1.
constexpr int64_t kMaxBlocks = 2147483647LL;

// rows and seqlen a call can have: non-negative, rows within the grid limit, and
// the byte size of a tensor (plus a tile of slack for index arithmetic) within int64.
bool shape_ok(int64_t rows, int64_t seqlen) {
    if (rows < 0 || seqlen < 0 || rows > kMaxBlocks) return false;
    return rows == 0 || seqlen <= (INT64_MAX >> 5) / rows;
}

bool activation_supported(int act, int dtype, bool reverse) {
    if (act == ASCAN_GATE_IDENTITY) return true;
    return (act == ASCAN_GATE_SIGMOID || act == ASCAN_GATE_SIGMOID_LERP || act == ASCAN_GATE_EXP ||
            act == ASCAN_GATE_EXP_NORM) && !reverse &&
           (dtype == ASCAN_F32 || dtype == ASCAN_BF16 || dtype == ASCAN_F16);
}
static_assert(ASCAN_GATE_IDENTITY == kGateIdentity && ASCAN_GATE_SIGMOID == kGateSigmoid &&
                  ASCAN_GATE_SIGMOID_LERP == kGateSigmoidLerp && ASCAN_GATE_EXP == kGateExp &&
                  ASCAN_GATE_EXP_NORM == kGateExpNorm,
              "the kernels' gate codes are the ABI's");

int forward_checked(const void* gates, const void* tokens, void* out, const void* initial, int64_t rows,
                    int64_t seqlen, int dtype, int reverse, int act, const Workspace& ws, void* stream) {
    const size_t es = element_size(dtype);
    if (es == 0) return ASCAN_ERR_BAD_DTYPE;
    if (!activation_supported(act, dtype, reverse != 0)) return ASCAN_ERR_BAD_ACTIVATION;
    if (!shape_ok(rows, seqlen)) return ASCAN_ERR_BAD_SHAPE;
    if (rows == 0 || seqlen == 0) return ASCAN_OK;
    if (!gates || !tokens || !out) return ASCAN_ERR_NULL_POINTER;
    if (!element_aligned(gates, es) || !element_aligned(tokens, token_size(dtype)) || !element_aligned(out, es) ||
        !element_aligned(initial, es))
        return ASCAN_ERR_MISALIGNED;
    {
        const int64_t n = rows * seqlen;
        const Span inputs[] = {span_of(gates, n, es), span_of(tokens, n, token_size(dtype)), span_of(initial, rows, es)};
        const Span outputs[] = {span_of(out, n, es)};
        if (outputs_overlap(inputs, outputs)) return ASCAN_ERR_OVERLAP;
    }
    const ForwardCall call{gates, tokens, out, initial, rows, seqlen, reverse != 0, act, ws,
                           static_cast<hipStream_t>(stream)};
    switch (dtype) {
        case ASCAN_F32: return forward_f32(call);
        case ASCAN_BF16: return forward_bf16(call);
        case ASCAN_F16: return forward_f16(call);
        case ASCAN_C64: return forward_c64(call);
        default: return forward_c64_real_tokens(call);
    }
}

// `values` is the fourth input of the gates with values and null for every other gate;
// `reverse` says that the scan being differentiated ran backwards in time (identity gate only).
int backward_checked(const void* gates, const void* states, const void* grad_out, void* d_gates, void* d_tokens,
                     const void* initial, void* d_initial, const void* values, int64_t rows, int64_t seqlen,
                     int dtype, int act, bool reverse, const Workspace& ws, void* stream) {
    const size_t es = element_size(dtype);
    if (es == 0) return ASCAN_ERR_BAD_DTYPE;
    if (!activation_supported(act, dtype, reverse)) return ASCAN_ERR_BAD_ACTIVATION;
    if (!shape_ok(rows, seqlen)) return ASCAN_ERR_BAD_SHAPE;
    if (rows == 0 || seqlen == 0) return ASCAN_OK;
    if (!gates || !states || !grad_out || !d_gates || !d_tokens) return ASCAN_ERR_NULL_POINTER;
    if (gate_takes_values(act) && !values) return ASCAN_ERR_NULL_POINTER;
    if (!element_aligned(gates, es) || !element_aligned(states, es) || !element_aligned(grad_out, es) ||
        !element_aligned(d_gates, es) || !element_aligned(d_tokens, token_size(dtype)) ||
        !element_aligned(initial, es) || !element_aligned(d_initial, es) || !element_aligned(values, es))
        return ASCAN_ERR_MISALIGNED;
    {
        const int64_t n = rows * seqlen;
        const Span inputs[] = {span_of(gates, n, es), span_of(states, n, es), span_of(grad_out, n, es),
                               span_of(initial, rows, es), span_of(values, n, es)};
        const Span outputs[] = {span_of(d_gates, n, es), span_of(d_tokens, n, token_size(dtype)),
                                span_of(d_initial, rows, es)};
        if (outputs_overlap(inputs, outputs)) return ASCAN_ERR_OVERLAP;
    }
    const BackwardCall call{gates, states, grad_out, d_gates, d_tokens, initial, d_initial, values, rows, seqlen, act,
                            ws, static_cast<hipStream_t>(stream)};
    if (reverse) {
        switch (dtype) {
            case ASCAN_F32: return backward_reverse_f32(call);
            case ASCAN_BF16: return backward_reverse_bf16(call);
            case ASCAN_F16: return backward_reverse_f16(call);
            case ASCAN_C64: return backward_reverse_c64(call);
            default: return backward_reverse_c64_real_tokens(call);
        }
    }
    switch (dtype) {
        case ASCAN_F32: return backward_f32(call);
        case ASCAN_BF16: return backward_bf16(call);
        case ASCAN_F16: return backward_f16(call);
        case ASCAN_C64: return backward_c64(call);
        default: return backward_c64_real_tokens(call);
    }
}

}  // namespace
}  // namespace ascan

using namespace ascan;

extern "C" {

int ascan_forward(const void* gates, const void* tokens, void* out, int64_t rows, int64_t seqlen, int dtype,
                  int reverse, void* stream) {
    return forward_checked(gates, tokens, out, nullptr, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY,
                           Workspace{nullptr, 0}, stream);
}

int ascan_backward(const void* gates, const void* states, const void* grad_out, void* d_gates, void* d_tokens,
                   int64_t rows, int64_t seqlen, int dtype, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, nullptr, nullptr, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, false, Workspace{nullptr, 0}, stream);
}

namespace {
// Size of the table for a call (`forward_only`: for the identity gate's forward kernel alone).
size_t table_bytes(int64_t rows, int64_t seqlen, int dtype, bool forward_only) {
    const size_t es = element_size(dtype);
    if (es == 0 || rows <= 0 || seqlen <= 0 || !shape_ok(rows, seqlen)) return 0;
    // the smallest split tile any kernel uses for this dtype: 2 blocks of 64 vectors per wave
    const int64_t epv = 16 / (int64_t)es;
    const int64_t tile = (int64_t)kSplitWaves * 2 * 64 * epv;
    // rows are addressed from the 128-byte boundary below their first element at most
    const int64_t head = 128 / (int64_t)es - 1;
    const int64_t ntiles = (seqlen + head + tile - 1) / tile;
    const SweepClass c = dtype == ASCAN_F32 ? SweepClass::kF32
                         : (dtype == ASCAN_BF16 || dtype == ASCAN_F16 ? SweepClass::kNarrow : SweepClass::kComplex);
    if (may_split(c, rows, seqlen * (int64_t)es, ntiles, forward_only) && rows <= 2147483647LL / ntiles) {
        return split_bytes(rows, ntiles);
    }
    if (forward_only && forward_needs_ticket_only(c, rows, seqlen * (int64_t)es)) return split_bytes(0, 1);
    return 0;
}
}  // namespace

size_t ascan_workspace_bytes(int64_t rows, int64_t seqlen, int dtype) { return table_bytes(rows, seqlen, dtype, false); }

int ascan_forward_split(const void* gates, const void* tokens, void* out, int64_t rows, int64_t seqlen, int dtype,
                        int reverse, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_checked(gates, tokens, out, nullptr, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY,
                           Workspace{workspace, workspace_bytes}, stream);
}

int ascan_forward_split_static(const void* gates, const void* tokens, void* out, int64_t rows, int64_t seqlen,
                               int dtype, int reverse, void* stream) {
    // what this call's one kernel may use: less than ascan_workspace_bytes where only a backward kernel is swept
    const size_t needed = table_bytes(rows, seqlen, dtype, true);
    if (needed > (size_t)ASCAN_STATIC_WORKSPACE_BYTES) return ASCAN_ERR_TOO_LARGE;
    Workspace ws{nullptr, 0};
    // needed == 0: rows that are not split (or arguments the checks below refuse) use no table
    if (needed != 0 && gates && tokens && out) {
        ws.ptr = static_workspace();
        if (ws.ptr == nullptr) return ASCAN_ERR_LAUNCH;
        ws.bytes = (size_t)ASCAN_STATIC_WORKSPACE_BYTES;
    }
    return forward_checked(gates, tokens, out, nullptr, rows, seqlen, dtype, reverse, ASCAN_GATE_IDENTITY, ws, stream);
}

int ascan_static_workspace_timeouts(unsigned int* count, void* stream) {
    if (count == nullptr) return ASCAN_ERR_NULL_POINTER;
    void* table = static_workspace();
    if (table == nullptr) return ASCAN_ERR_LAUNCH;
    SplitHeader header;
    hipError_t e = hipStreamSynchronize(static_cast<hipStream_t>(stream));
    if (e == hipSuccess) e = hipMemcpy(&header, table, sizeof(header), hipMemcpyDeviceToHost);
    if (e != hipSuccess) {
        g_last_hip_error = (int)e;
        return ASCAN_ERR_LAUNCH;
    }
    *count = header.timeouts;
    return ASCAN_OK;
}

int ascan_backward_split(const void* gates, const void* states, const void* grad_out, void* d_gates,
                         void* d_tokens, int64_t rows, int64_t seqlen, int dtype, void* workspace,
                         size_t workspace_bytes, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, nullptr, nullptr, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, false, Workspace{workspace, workspace_bytes}, stream);
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
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, false, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_reverse(const void* gates, const void* states, const void* initial, const void* grad_out,
                           void* d_gates, void* d_tokens, void* d_initial, int64_t rows, int64_t seqlen, int dtype,
                           void* workspace, size_t workspace_bytes, void* stream) {
    return backward_checked(gates, states, grad_out, d_gates, d_tokens, initial, d_initial, nullptr, rows, seqlen, dtype,
                            ASCAN_GATE_IDENTITY, true, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_forward_gated(const void* gate_inputs, const void* tokens, const void* initial, void* out, int64_t rows,
                        int64_t seqlen, int dtype, int gate, void* workspace, size_t workspace_bytes, void* stream) {
    return forward_checked(gate_inputs, tokens, out, initial, rows, seqlen, dtype, 0, gate,
                           Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_gated(const void* gate_inputs, const void* states, const void* initial, const void* grad_out,
                         void* d_gate_inputs, void* d_tokens, void* d_initial, int64_t rows, int64_t seqlen,
                         int dtype, int gate, void* workspace, size_t workspace_bytes, void* stream) {
    if (gate_takes_values(gate)) return ASCAN_ERR_BAD_ACTIVATION;  // needs the values: ascan_backward_gated_values
    return backward_checked(gate_inputs, states, grad_out, d_gate_inputs, d_tokens, initial, d_initial, nullptr, rows,
                            seqlen, dtype, gate, false, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_lerp(const void* gate_inputs, const void* values, const void* states, const void* initial,
                        const void* grad_out, void* d_gate_inputs, void* d_values, void* d_initial, int64_t rows,
                        int64_t seqlen, int dtype, void* workspace, size_t workspace_bytes, void* stream) {
    return backward_checked(gate_inputs, states, grad_out, d_gate_inputs, d_values, initial, d_initial, values, rows,
                            seqlen, dtype, ASCAN_GATE_SIGMOID_LERP, false, Workspace{workspace, workspace_bytes}, stream);
}

int ascan_backward_gated_values(const void* gate_inputs, const void* values, const void* states, const void* initial,
                                const void* grad_out, void* d_gate_inputs, void* d_values, void* d_initial,
                                int64_t rows, int64_t seqlen, int dtype, int gate, void* workspace,
                                size_t workspace_bytes, void* stream) {
    if (!gate_takes_values(gate)) return ASCAN_ERR_BAD_ACTIVATION;
    return backward_checked(gate_inputs, states, grad_out, d_gate_inputs, d_values, initial, d_initial, values, rows,
                            seqlen, dtype, gate, false, Workspace{workspace, workspace_bytes}, stream);
}

unsigned int ascan_workspace_timeouts(const void* workspace_header_copy) {
    return static_cast<const SplitHeader*>(workspace_header_copy)->timeouts;
}

const char* ascan_status_string(int status) {
    switch (status) {
        case ASCAN_OK: return "ok";
        case ASCAN_ERR_NULL_POINTER: return "a required buffer pointer is NULL";
        case ASCAN_ERR_BAD_SHAPE: return "rows or seqlen is negative, rows exceeds the grid limit, or rows * seqlen does not fit the address space";
        case ASCAN_ERR_BAD_DTYPE: return "unsupported dtype: expecting float32, bfloat16, float16, complex64 or complex64 with float32 tokens";
        case ASCAN_ERR_MISALIGNED: return "a buffer is not aligned to its element size";
        case ASCAN_ERR_LAUNCH: return "the HIP runtime reported a launch error";
        case ASCAN_ERR_BAD_ACTIVATION:
            return "unsupported gate activation: expecting identity, or a sigmoid or exponential gate with float32, bfloat16 or float16";
        case ASCAN_ERR_OVERLAP: return "an output buffer overlaps an input or another output buffer of the call";
        case ASCAN_ERR_TOO_LARGE:
            return "the split-row table of this problem exceeds the library's static workspace (ASCAN_STATIC_WORKSPACE_BYTES)";
        default: return "unknown status";
    }
}

int ascan_last_hip_error(void) { return g_last_hip_error; }

int ascan_abi_version(void) { return ASCAN_ABI_VERSION; }

}  // extern "C"
