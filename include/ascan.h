/*
 * ascan.h -- C ABI of the MI355X (gfx950) first-order scan library.
 *
 * The library solves, independently for every row of a contiguous
 * (rows, seqlen) matrix (rows = B*D of a (B, D, T) tensor, T innermost):
 *
 *     forward :  x[t] = gate[t] * x[t-1] + token[t],      x[-1] = 0
 *     reverse :  y[t] = gate[t] * y[t+1] + token[t],      y[T]  = 0
 *     backward:  g[t] = grad_out[t] + conj(gate[t+1]) * g[t+1],   g[T] = 0
 *                d_tokens[t] = g[t]
 *                d_gates[t]  = g[t] * conj(x[t-1]),       x[-1] = 0
 *
 * (conj is the identity for the real dtypes).
 *
 * These entry points stand where the reference binds its compiled extension:
 *   accelerated_scan/warp.py:29-30   (module.warpscan_forward / warpscan_backward)
 *   accelerated_scan/warp.cuh:394-424 (the two functions those names resolve to)
 * and, for ASCAN_C64, where accelerated_scan/complex.py:174-180,205-214 launches
 * its forward_scan / backward_scan kernels.
 *
 * Conventions
 *   - every buffer is device memory owned by the caller; the library allocates
 *     nothing, keeps no reference after the call returns and holds no mutable
 *     global state, so calls are re-entrant from any host thread (the *_split
 *     calls additionally need a caller-provided workspace per concurrent call);
 *   - kernels are launched on the calling thread's CURRENT HIP device: every
 *     pointer of a call (buffers, workspace) must be memory of that device and
 *     `stream` a stream of that device.  The library does not look the pointers
 *     up; a caller with several GPUs makes the right one current first
 *     (hipSetDevice), as the Python binding does;
 *   - work is enqueued on `stream` (a hipStream_t passed as void*, NULL = the
 *     default stream) and the call returns without synchronising;
 *   - rows are dense: row r starts at element r*seqlen; 64-bit element offsets
 *     are used throughout, so rows*seqlen may exceed 2^31;
 *   - no output buffer may overlap an input buffer or another output buffer of
 *     the same call (the kernels read and write rows in tiles, out of order
 *     across workgroups): such a call is refused with ASCAN_ERR_OVERLAP and
 *     nothing is launched;
 *   - rows shorter than 2 KiB are scanned several to a workgroup, as one long
 *     sequence with a zero gate inserted in front of every row.  In that mode a
 *     gate of exactly zero discards the state it multiplies even when that state
 *     is not finite (0 * inf counts as 0, not NaN), for the inserted zeros and
 *     for zeros stored in `gates` alike; for longer rows, as in the reference,
 *     a stored zero gate times a non-finite state is NaN.  Finite data is not
 *     affected;
 *   - arithmetic is done in fp32 for every dtype (bf16/fp16 are storage
 *     formats, rounded to nearest-even on store);
 *   - buffers whose addresses agree modulo 16 (the usual case: allocator
 *     blocks, or equal storage offsets) take the vectorised kernels for any
 *     seqlen, at full speed when they also agree modulo 128; buffers at
 *     different offsets inside a 16-byte block take element-wise kernels with
 *     the same arithmetic.  The vectorised kernels move aligned 16-byte blocks
 *     only: where a tensor does not begin or end on a 16-byte boundary they READ
 *     the whole block that straddles its first or last element, i.e. up to 15
 *     bytes outside the tensor's range (inside the same 16-byte block, so inside
 *     the same page and allocation granule), and discard them; they never write
 *     outside the range.  A caller that sub-allocates tensors at odd offsets while
 *     another stream writes the neighbouring bytes will see those reads in a race
 *     detector; the results do not depend on them;
 *   - results are reproducible: the same call on the same data gives the same
 *     bits, run to run and whatever else the GPU is doing, on every path
 *     (including rows split over workgroups, see below);
 *   - errors are reported by return code, never by abort or exception.
 */
#ifndef ASCAN_H_
#define ASCAN_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define ASCAN_ABI_VERSION 10

/* Marks the exported entry points (the library is built with hidden visibility). */
#define ASCAN_API __attribute__((visibility("default")))

/* Element types of the tensors of a call. */
enum ascan_dtype {
    ASCAN_F32  = 0, /* float                                   (warp.cuh:388) */
    ASCAN_BF16 = 1, /* bfloat16 storage, fp32 arithmetic       (warp.cuh:384) */
    ASCAN_F16  = 2, /* IEEE half storage, fp32 arithmetic      (warp.cuh:386) */
    ASCAN_C64  = 3, /* complex64 = interleaved (re, im) floats (complex.py:37-42) */
    /*
     * complex64 gates, states, grad_out and d_gates with float tokens and
     * d_tokens: the case complex.scan accepts by promoting real inputs to a
     * complex copy and keeping the real part of their gradient
     * (complex.py:162,168-169,217-218).  Here the tokens are read as
     * (token, 0) and d_tokens receives Re g[t]; no complex copy is made.
     */
    ASCAN_C64_REAL_TOKENS = 4
};

/* Return codes. */
enum ascan_status {
    ASCAN_OK                = 0,
    ASCAN_ERR_NULL_POINTER  = 1, /* a required buffer is NULL while rows*seqlen > 0 */
    ASCAN_ERR_BAD_SHAPE     = 2, /* rows < 0, seqlen < 0, rows too large for one grid, or rows * seqlen beyond 2^58 */
    ASCAN_ERR_BAD_DTYPE     = 3, /* dtype is not an ascan_dtype (warp.cuh:390-391) */
    ASCAN_ERR_MISALIGNED    = 4, /* a pointer is not aligned to its element size */
    ASCAN_ERR_LAUNCH        = 5, /* the HIP runtime refused the launch (see ascan_last_hip_error) */
    ASCAN_ERR_BAD_ACTIVATION = 6, /* gate is not an ascan_gate, or not available for this dtype */
    ASCAN_ERR_OVERLAP       = 7, /* an output buffer overlaps an input or another output of the call */
    ASCAN_ERR_TOO_LARGE     = 8  /* ascan_forward_split_static: the table would not fit the static workspace */
};

/* What the kernels make of the stored gate values (the *_gated entry points). */
enum ascan_gate {
    ASCAN_GATE_IDENTITY = 0, /* stored values are the gates: the reference's operator */
    ASCAN_GATE_SIGMOID  = 1, /* gate = 1 / (1 + exp(-stored)); float32, bfloat16, float16 */
    /*
     * The same gate, and the second input holds values v rather than tokens:
     * token = (1 - gate) * v, i.e. x[t] = gate * x[t-1] + (1 - gate) * v[t], the
     * gated interpolation of linear-RNN layers.  Forward: ascan_forward_gated;
     * backward: ascan_backward_lerp (it needs v).  float32, bfloat16, float16.
     */
    ASCAN_GATE_SIGMOID_LERP = 2,
    /*
     * gate = exp(stored): the stored values are logarithms of the gates (decay
     * rates; <= 0 for gates in (0, 1]).  A 16-bit logarithm holds a gate close
     * to 1 far more precisely than a 16-bit gate can (bfloat16 has no value
     * between 0.99609375 and 1).  float32, bfloat16, float16.
     */
    ASCAN_GATE_EXP = 3,
    /*
     * The same gate, and the second input holds values v rather than tokens:
     * token = sqrt(1 - gate^2) * v, i.e. x[t] = a * x[t-1] + sqrt(1 - a^2) * v[t]
     * with a = exp(stored), the update of RG-LRU / Hawk-style layers (the scale
     * keeps the state's variance at that of the values).  Stored values should be
     * negative: at 0 the scale is 0 and its derivative unbounded; the backward
     * pass takes the derivative of the scale as 0 there (a stored +0 or -0, e.g. a
     * 16-bit logarithm that underflowed), so gradients stay finite.  Forward:
     * ascan_forward_gated; backward: ascan_backward_gated_values (it needs v).
     * float32, bfloat16, float16.
     */
    ASCAN_GATE_EXP_NORM = 4
};

/*
 * Replaces warpscan_forward (accelerated_scan/warp.cuh:394-405; bound at
 * warp.py:29) and the forward_scan launches at scalar.py:98 and
 * complex.py:174-180.  out[r, t] receives the inclusive scan of row r.
 * reverse != 0 runs the recurrence from t = seqlen-1 down to 0 with the
 * un-shifted gates (the `reverse` argument of warp.cuh:395).
 */
ASCAN_API int ascan_forward(const void* gates, const void* tokens, void* out,
                  int64_t rows, int64_t seqlen, int dtype, int reverse,
                  void* stream);

/*
 * Replaces warpscan_backward (accelerated_scan/warp.cuh:407-424; bound at
 * warp.py:30) and the backward_scan launches at scalar.py:116-124 and
 * complex.py:205-214.  `states` is the forward output, `grad_out` the incoming
 * gradient; d_gates and d_tokens receive the two gradients.  One fused
 * reverse-time pass: 3 tensors read, 2 written.
 */
ASCAN_API int ascan_backward(const void* gates, const void* states, const void* grad_out,
                   void* d_gates, void* d_tokens,
                   int64_t rows, int64_t seqlen, int dtype,
                   void* stream);

/*
 * Rows split over workgroups, with a table in caller-provided memory.  The
 * plain entry points give every row to one workgroup that walks it from end
 * to end.  That leaves most of the GPU idle when there are few rows, and for
 * long rows it is not the fastest order either: with thousands of rows being
 * walked side by side the memory system sees as many streams.  Given a
 * workspace, the *_split entry points (and every entry point below that takes
 * one) instead hand out the 16-wave tiles of all rows in memory order, one
 * tile at a time to whichever resident workgroup is free, and pass the running
 * state from tile to tile through a small table in the workspace: one pass over
 * the data, no extra traffic.  Measured on MI355X, fp32 (8, 1536, 65536) forward +
 * backward: 4.40 ms without a workspace, 3.90 ms with one.  (Rows of exactly half
 * a tile -- 32 KiB, starting on a 128-byte boundary -- are swept as well once the
 * tensors reach 256 MiB, two whole rows to a tile; the table then serves for the
 * ticket only.)  They have no
 * counterpart in the reference, whose kernels give one thread block to each
 * sequence (warp.cuh:279; scalar.py:98; complex.py:174).
 *
 *   ascan_workspace_bytes  size of the table for a problem, or 0 when no kernel
 *                          would use one (short rows; complex64 rows beyond
 *                          512 KiB unless they are few): then the calls behave
 *                          exactly like the plain ones and ignore the workspace.
 *                          Which kernels of a shape are swept is decided per
 *                          kernel (of complex64 and of the 16-bit gates with a
 *                          sigmoid, the backward kernel only).  Otherwise 128 bytes plus 64
 *                          bytes per tile, a few MB at most for tensors of GBs;
 *   workspace              device memory, 64-byte aligned, at least that many
 *                          bytes, not shared with another call that may run at
 *                          the same time; contents on entry do not matter (it
 *                          is cleared by a small kernel on `stream` first) and
 *                          it may be freed or reused once the work on `stream`
 *                          has completed.  NULL or a too-small buffer selects
 *                          the plain path.
 *
 * A workgroup waits for the workgroups of earlier tiles of its row.  Tiles are
 * handed out in order by one ticket counter, and a workgroup starts on its tile
 * as soon as it has drawn the ticket, so the owner of a tile that is waited
 * for has always started already: progress does not depend on how much of the
 * GPU the call gets, and concurrent calls (each with its own workspace) are
 * fine.  What a tile receives is the state entering its window of 64 tiles
 * folded with the aggregates of the window's earlier tiles in one fixed order,
 * whichever of them were published first: results are the same bits run to run
 * (they differ from the plain path's by rounding, the association being another).
 * Every wait is bounded all the same (2 s of running time by default; the
 * environment variable ASCAN_SPLIT_WAIT_US, read once, sets another limit); a
 * wait that runs out writes NaN into the affected tile and is counted: copy
 * the first 64 bytes of the workspace to the host after the stream has
 * completed and pass them to ascan_workspace_timeouts (0 = all waits were
 * served).  NaN in whole tiles of an output whose inputs are finite means that
 * a wait ran out.
 */
ASCAN_API size_t ascan_workspace_bytes(int64_t rows, int64_t seqlen, int dtype);

ASCAN_API int ascan_forward_split(const void* gates, const void* tokens, void* out,
                        int64_t rows, int64_t seqlen, int dtype, int reverse,
                        void* workspace, size_t workspace_bytes, void* stream);

ASCAN_API int ascan_backward_split(const void* gates, const void* states, const void* grad_out,
                         void* d_gates, void* d_tokens,
                         int64_t rows, int64_t seqlen, int dtype,
                         void* workspace, size_t workspace_bytes, void* stream);

ASCAN_API unsigned int ascan_workspace_timeouts(const void* workspace_header_copy);

/*
 * ascan_forward_split for callers that cannot allocate device memory at all
 * (code running under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc): the split-row table lives in a static device-side array
 * inside the library instead of a caller-provided workspace, and the call
 * allocates nothing, on the host side or the device side.  It has no
 * counterpart in the reference.  Results are those of ascan_forward_split.
 *
 *   - the array holds ASCAN_STATIC_WORKSPACE_BYTES on every GPU the library is
 *     used on, from the first call on that GPU until the process ends;
 *   - a problem whose table would be larger is refused with ASCAN_ERR_TOO_LARGE
 *     and nothing is launched.  The table meant is that of this call's one
 *     kernel, the identity gate's forward kernel: at most ascan_workspace_bytes,
 *     and less where only a backward kernel of the shape would be swept.
 *     Problems whose forward kernel is not swept run the plain kernel and use
 *     no table;
 *   - all calls on one GPU share that GPU's array (it is cleared by a small
 *     kernel on `stream` at the start of each call): two calls that may run at
 *     the same time on one GPU -- different streams, or graph branches -- race
 *     on it.  Use ascan_forward_split with separate workspaces for those;
 *   - the first use on a GPU looks the array's address up (hipGetSymbolAddress,
 *     which loads the library's code object on that GPU): make it outside any
 *     stream capture -- a first call of ascan_static_workspace_timeouts does.
 *
 * ascan_static_workspace_timeouts waits for `stream` and stores in *count the
 * number of waits that ran out in the last ascan_forward_split_static call on the
 * current GPU that used the table (see ascan_workspace_timeouts; whatever the
 * array holds before the first such call counts as 0 only if it is zero, which
 * it is at load time).  Not for use under capture.
 */
#define ASCAN_STATIC_WORKSPACE_BYTES (4 * 1024 * 1024)

ASCAN_API int ascan_forward_split_static(const void* gates, const void* tokens, void* out,
                               int64_t rows, int64_t seqlen, int dtype, int reverse,
                               void* stream);

ASCAN_API int ascan_static_workspace_timeouts(unsigned int* count, void* stream);

/*
 * Scans that start from a given state, for callers that process a long
 * sequence in chunks (streaming inference, truncated back-propagation): the
 * final state of one chunk, out[:, seqlen-1], is the `initial` of the next.
 *
 *     forward :  x[-1] = initial[row]       (reverse: y[seqlen] = initial[row])
 *     backward:  d_gates[0]     = g[0] * conj(initial[row])
 *                d_initial[row] = conj(gate[0]) * g[0]
 *
 * No counterpart in the reference, whose scans always start from zero
 * (warp.cuh:76 kEmptyToken, scalar.py:28 h0 and complex.py:32-33 state_x = zeros).
 *
 *   initial    `rows` elements of the dtype of `out` (complex64 for both complex
 *              dtypes), or NULL for zeros;
 *   d_initial  `rows` elements of that dtype, or NULL when the gradient is not
 *              wanted; not written when seqlen == 0;
 *   workspace  as for the *_split calls; NULL selects the plain path.
 *
 * With initial == NULL and d_initial == NULL these calls are the *_split ones.
 */
ASCAN_API int ascan_forward_from(const void* gates, const void* tokens, const void* initial, void* out,
                       int64_t rows, int64_t seqlen, int dtype, int reverse,
                       void* workspace, size_t workspace_bytes, void* stream);

ASCAN_API int ascan_backward_from(const void* gates, const void* states, const void* initial,
                        const void* grad_out, void* d_gates, void* d_tokens, void* d_initial,
                        int64_t rows, int64_t seqlen, int dtype,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward pass of a reverse scan, y[t] = gate[t] * y[t+1] + token[t] with
 * y[seqlen] = initial (NULL: 0), i.e. of ascan_forward / ascan_forward_from /
 * ascan_forward_split called with reverse != 0.  `states` is that call's output.
 *
 *     g[t]        = grad_out[t] + conj(gate[t-1]) * g[t-1]     (a forward-time scan, g[-1] = 0)
 *     d_tokens[t] = g[t]
 *     d_gates[t]  = g[t] * conj(y[t+1])                        (y[seqlen] = initial)
 *     d_initial   = conj(gate[seqlen-1]) * g[seqlen-1]
 *
 * One fused pass like ascan_backward, mirrored in time.  No counterpart in the
 * reference: its reverse scan (warp.py:32-35, the `reverse` argument of
 * warp.cuh:395) exists to compute gradients and is not differentiable itself;
 * layers that scan a sequence in both directions need this.  Arguments as for
 * ascan_backward_from; initial, d_initial and workspace may each be NULL.
 */
ASCAN_API int ascan_backward_reverse(const void* gates, const void* states, const void* initial,
                           const void* grad_out, void* d_gates, void* d_tokens, void* d_initial,
                           int64_t rows, int64_t seqlen, int dtype,
                           void* workspace, size_t workspace_bytes, void* stream);

/*
 * Scans whose gates come out of a non-linearity, applied in registers: the
 * caller passes the pre-activations and receives the gradient with respect to
 * them, instead of running one elementwise pass that materialises the gates and
 * another that turns d_gates into the gradient of the pre-activations (the
 * linear-RNN layers that call the scan, README.md:8,42 of the reference,
 * typically compute their gates with a sigmoid just before it).
 *
 *     gate[t]          = act(gate_inputs[t])
 *     forward          : x[t] = gate[t] * x[t-1] + tokens[t],   x[-1] = initial (NULL: 0)
 *     d_gate_inputs[t] = g[t] * x[t-1] * act'(gate_inputs[t])
 *
 * with g, d_tokens and d_initial as in ascan_backward_from.  No counterpart in
 * the reference.  gate = ASCAN_GATE_IDENTITY makes these calls the *_from ones
 * (forward in time only); the sigmoid and exponential gates need a real dtype, else
 * ASCAN_ERR_BAD_ACTIVATION (as do ASCAN_GATE_SIGMOID_LERP and ASCAN_GATE_EXP_NORM in
 * ascan_backward_gated, which lacks the values: see ascan_backward_gated_values).  The sigmoid is evaluated in fp32 with the
 * hardware's exp2 and reciprocal (about 2 ulp), the exponential with exp2 (1 ulp
 * of the result for arguments of moderate size).
 */
ASCAN_API int ascan_forward_gated(const void* gate_inputs, const void* tokens, const void* initial, void* out,
                        int64_t rows, int64_t seqlen, int dtype, int gate,
                        void* workspace, size_t workspace_bytes, void* stream);

ASCAN_API int ascan_backward_gated(const void* gate_inputs, const void* states, const void* initial,
                         const void* grad_out, void* d_gate_inputs, void* d_tokens, void* d_initial,
                         int64_t rows, int64_t seqlen, int dtype, int gate,
                         void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward pass of ascan_forward_gated(gate_inputs, values, ..., ASCAN_GATE_SIGMOID_LERP):
 *
 *     a[t]             = sigmoid(gate_inputs[t])
 *     forward          : x[t] = a[t] * x[t-1] + (1 - a[t]) * values[t],   x[-1] = initial (NULL: 0)
 *     g[t]             = grad_out[t] + a[t+1] * g[t+1]
 *     d_values[t]      = g[t] * (1 - a[t])
 *     d_gate_inputs[t] = g[t] * (x[t-1] - values[t]) * a[t] * (1 - a[t])
 *     d_initial        = a[0] * g[0]
 *
 * One fused reverse-time pass: 4 tensors read, 2 written (against 3 + 2 for the
 * scan alone plus three elementwise passes over 11 tensors for the token
 * product and its gradient when they are done outside).  1 - a is evaluated as
 * sigmoid(-gate_inputs), not as a difference.  No counterpart in the reference.
 */
ASCAN_API int ascan_backward_lerp(const void* gate_inputs, const void* values, const void* states, const void* initial,
                        const void* grad_out, void* d_gate_inputs, void* d_values, void* d_initial,
                        int64_t rows, int64_t seqlen, int dtype,
                        void* workspace, size_t workspace_bytes, void* stream);

/*
 * Backward pass of ascan_forward_gated for the gates whose second input holds
 * values: gate = ASCAN_GATE_SIGMOID_LERP is ascan_backward_lerp, and
 * gate = ASCAN_GATE_EXP_NORM differentiates
 *
 *     a[t] = exp(gate_inputs[t]),   b[t] = sqrt(1 - a[t]^2)
 *     forward          : x[t] = a[t] * x[t-1] + b[t] * values[t],   x[-1] = initial (NULL: 0)
 *     g[t]             = grad_out[t] + a[t+1] * g[t+1]
 *     d_values[t]      = g[t] * b[t]
 *     d_gate_inputs[t] = g[t] * (a[t] * x[t-1] - values[t] * a[t]^2 / b[t])
 *     d_initial        = a[0] * g[0]
 *
 * in one fused reverse-time pass (4 tensors read, 2 written).  1 - a^2 is
 * evaluated without cancellation for gates close to 1 (a series in
 * 2 * gate_inputs where that is above -1/16); where b is exactly 0
 * (gate_inputs = 0) the term values * a^2 / b is taken as 0.  Any other gate:
 * ASCAN_ERR_BAD_ACTIVATION.
 * No counterpart in the reference.
 */
ASCAN_API int ascan_backward_gated_values(const void* gate_inputs, const void* values, const void* states,
                                const void* initial, const void* grad_out, void* d_gate_inputs, void* d_values,
                                void* d_initial, int64_t rows, int64_t seqlen, int dtype, int gate,
                                void* workspace, size_t workspace_bytes, void* stream);

/* Static, human-readable text for an ascan_status code. */
ASCAN_API const char* ascan_status_string(int status);

/* hipError_t (as int) recorded by the calling thread's last ASCAN_ERR_LAUNCH. */
ASCAN_API int ascan_last_hip_error(void);

/* ASCAN_ABI_VERSION the library was built with. */
ASCAN_API int ascan_abi_version(void);

#ifdef __cplusplus
}
#endif

#endif /* ASCAN_H_ */
