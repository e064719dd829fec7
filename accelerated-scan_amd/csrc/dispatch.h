// What the C entry points (ascan.hip) call: one forward function and two backward
// functions (for forward-time and for reverse scans) per dtype, each compiled in a
// translation unit of its own (forward_<dtype>.hip, backward_<dtype>.hip,
// backward_reverse_<dtype>.hip) together with its kernels.
#ifndef ASCAN_DISPATCH_H_
#define ASCAN_DISPATCH_H_

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace ascan {

// Caller-provided table for split rows (may be absent).
struct Workspace {
    void* ptr;
    size_t bytes;
};

// Arguments of a forward call after validation (device pointers, rows x seqlen elements).
struct ForwardCall {
    const void* gates;    // or gate pre-activations, see `gate`
    const void* tokens;
    void* out;
    const void* initial;  // one state per row, or null
    int64_t rows, seqlen;
    bool reverse;
    int gate;             // ascan_gate
    Workspace workspace;
    hipStream_t stream;
};

struct BackwardCall {
    const void* gates;
    const void* states;
    const void* grad_out;
    void* d_gates;
    void* d_tokens;
    const void* initial;  // or null
    void* d_initial;      // or null
    const void* values;   // values v of a gate with values (then d_tokens receives d_v), else null
    int64_t rows, seqlen;
    int gate;
    Workspace workspace;
    hipStream_t stream;
};

// Each returns an ascan_status.
int forward_f32(const ForwardCall& call);
int forward_bf16(const ForwardCall& call);
int forward_f16(const ForwardCall& call);
int forward_c64(const ForwardCall& call);
int forward_c64_real_tokens(const ForwardCall& call);
int backward_f32(const BackwardCall& call);
int backward_bf16(const BackwardCall& call);
int backward_f16(const BackwardCall& call);
int backward_c64(const BackwardCall& call);
int backward_c64_real_tokens(const BackwardCall& call);
// Backward passes of reverse scans (identity gate only).
int backward_reverse_f32(const BackwardCall& call);
int backward_reverse_bf16(const BackwardCall& call);
int backward_reverse_f16(const BackwardCall& call);
int backward_reverse_c64(const BackwardCall& call);
int backward_reverse_c64_real_tokens(const BackwardCall& call);

// hipError_t of the calling thread's last failed launch (defined in ascan.hip).
extern thread_local int g_last_hip_error;

}  // namespace ascan

#endif  // ASCAN_DISPATCH_H_
