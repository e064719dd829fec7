"""ctypes binding of the HIP scan library (C ABI in ``include/ascan.h``).

This is the only place that touches the shared library.  There is no fallback:
if ``libascan.so`` is missing, ``load()`` raises, and so does every operator
built on it.  The library is searched for next to this file, or at the path in
the ``ASCAN_LIBRARY`` environment variable.
"""

import ctypes
import functools
import os
from pathlib import Path

import torch

ABI_VERSION = 10

# ascan_gate codes of include/ascan.h
GATE_IDENTITY, GATE_SIGMOID, GATE_SIGMOID_LERP, GATE_EXP, GATE_EXP_NORM = 0, 1, 2, 3, 4
# gates whose second input holds values: the backward pass reads them again
GATES_WITH_VALUES = (GATE_SIGMOID_LERP, GATE_EXP_NORM)

# ascan_dtype codes of include/ascan.h
F32, BF16, F16, C64, C64_REAL_TOKENS = 0, 1, 2, 3, 4

DTYPE_CODES = {
    torch.float32: F32,
    torch.bfloat16: BF16,
    torch.float16: F16,
    torch.complex64: C64,
}

_SIGNATURES = {
    # name: (restype, argtypes)
    "ascan_forward": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "ascan_backward": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_void_p],
    ),
    "ascan_workspace_bytes": (ctypes.c_size_t, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int]),
    "ascan_forward_split": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_split": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_workspace_timeouts": (ctypes.c_uint, [ctypes.c_void_p]),
    "ascan_forward_split_static": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    ),
    "ascan_static_workspace_timeouts": (ctypes.c_int, [ctypes.POINTER(ctypes.c_uint), ctypes.c_void_p]),
    "ascan_forward_from": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_from": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_reverse": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_forward_gated": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_gated": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_lerp": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_backward_gated_values": (
        ctypes.c_int,
        [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p,
         ctypes.c_int64, ctypes.c_int64, ctypes.c_int, ctypes.c_int,
         ctypes.c_void_p, ctypes.c_size_t, ctypes.c_void_p],
    ),
    "ascan_status_string": (ctypes.c_char_p, [ctypes.c_int]),
    "ascan_last_hip_error": (ctypes.c_int, []),
    "ascan_abi_version": (ctypes.c_int, []),
}

_lib = None


def library_path() -> Path:
    override = os.environ.get("ASCAN_LIBRARY")
    if override:
        return Path(override)
    return Path(__file__).resolve().parent / "libascan.so"


def load() -> ctypes.CDLL:
    """Load the shared library once and declare its prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    path = library_path()
    if not path.exists():
        raise ImportError(
            f"accelerated_scan: HIP library not found at {path}; build it with "
            f"`make -C {Path(__file__).resolve().parent.parent}` (needs hipcc, targets gfx950)"
        )
    lib = ctypes.CDLL(str(path))
    for name, (restype, argtypes) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    version = lib.ascan_abi_version()
    if version != ABI_VERSION:
        raise ImportError(f"accelerated_scan: {path} has ABI version {version}, expected {ABI_VERSION}")
    _lib = lib
    return lib


def exported_symbols():
    """Names the binding expects the library to export."""
    return tuple(_SIGNATURES)


def check(status: int) -> None:
    """Turn a non-zero ascan_status into RuntimeError (the reference raises
    RuntimeError through TORCH_CHECK, accelerated_scan/warp.cuh:379,391,396-421)."""
    if status == 0:
        return
    lib = load()
    text = lib.ascan_status_string(status).decode()
    if status == 5:
        text += f" (hipError_t {lib.ascan_last_hip_error()})"
    raise RuntimeError(f"accelerated_scan: {text}")


def dtype_code(dtype: torch.dtype, token_dtype: torch.dtype = None) -> int:
    """ascan_dtype of a call from the dtype of gates and of tokens / d_tokens."""
    if dtype == torch.complex64 and token_dtype == torch.float32:
        return C64_REAL_TOKENS
    if token_dtype is not None and token_dtype != dtype:
        raise RuntimeError(
            f"accelerated_scan: gates are {dtype} but tokens are {token_dtype}: expecting one dtype "
            "(or complex64 gates with float32 tokens)"
        )
    try:
        return DTYPE_CODES[dtype]
    except KeyError:
        raise RuntimeError(
            f"accelerated_scan: unsupported tensor dtype {dtype}: "
            "expecting bfloat16, float16, float32 or complex64"
        ) from None


def _stream_handle(index: int) -> int:
    """hipStream_t of torch's current stream on device ``index`` as an integer."""
    return torch.cuda.current_stream(index).cuda_stream


# torch keeps direct accessors for the current stream's handle (what its own
# compiled kernels launch on) and for the current device; they skip building
# Stream / device objects, several microseconds per call that matter for short
# sequences.
_stream_handle = getattr(torch._C, "_cuda_getCurrentRawStream", _stream_handle)
_current_device = getattr(torch._C, "_cuda_getDevice", torch.cuda.current_device)


def _launch(device: torch.device, fn, *args) -> None:
    """Call ``fn(*args, stream_handle)`` with ``device`` current (kernels launch on
    the current device, on torch's current stream there) and map the status."""
    index = device.index
    if index is None or index == _current_device():
        status = fn(*args, _stream_handle(_current_device() if index is None else index))
    else:
        with torch.cuda.device(index):
            status = fn(*args, _stream_handle(index))
    if status:
        check(status)


# ASCAN_DEBUG_SPLIT=1: after every call that was given a table, wait for the device and
# raise if a wait for an earlier tile ran out (such a tile holds NaN in the output).
_DEBUG_SPLIT = os.environ.get("ASCAN_DEBUG_SPLIT", "0") not in ("", "0")


def _after_split(workspace, what: str) -> None:
    if _DEBUG_SPLIT and workspace is not None:
        ran_out = workspace_timeouts(workspace)
        if ran_out:
            raise RuntimeError(f"accelerated_scan: {ran_out} wait(s) for an earlier tile ran out in {what}; "
                               "the affected tiles of the output hold NaN")


@functools.lru_cache(maxsize=1024)
def _workspace_bytes(rows: int, seqlen: int, code: int) -> int:
    return (_lib or load()).ascan_workspace_bytes(rows, seqlen, code)


def _workspace(rows: int, seqlen: int, code: int, device: torch.device):
    """Table for split rows (few rows, long sequences), or None.  Freed by the
    caching allocator in stream order after the kernels that use it."""
    nbytes = _workspace_bytes(rows, seqlen, code)
    if nbytes == 0:
        return None
    # (zeroed under ASCAN_DEBUG_SPLIT: a kernel that decides against the table leaves its header as it was)
    make = torch.zeros if _DEBUG_SPLIT else torch.empty
    return make(nbytes, dtype=torch.uint8, device=device)


def _check_state(state, like, name: str) -> None:
    """``initial`` / ``d_initial``: one element per row, in the dtype of the states."""
    if state is None:
        return
    if (not state.is_cuda or state.device != like.device or state.dtype != like.dtype
            or state.shape != like.shape[:-1] or not state.is_contiguous()):
        raise RuntimeError(
            f"accelerated_scan: expected {name} to be a contiguous {like.dtype} tensor of shape "
            f"{tuple(like.shape[:-1])} on {like.device}"
        )


def _problem(like, token_like):
    """(rows, seqlen, ascan_dtype) of a call from a state-like and a token-like tensor."""
    seqlen = like.shape[-1]
    rows = like.numel() // seqlen if seqlen else 0
    dtype, token_dtype = like.dtype, token_like.dtype
    code = DTYPE_CODES.get(dtype) if dtype == token_dtype else None
    if code is None:
        code = dtype_code(dtype, token_dtype)
    return rows, seqlen, code


def _ptr(t):
    return t.data_ptr() if t is not None else None


def forward(gates, tokens, out, reverse: bool, workspace=None, initial=None) -> None:
    """Enqueue the forward scan on the current stream of the tensors' device.
    ``initial`` (one state per row) starts the scan from that state."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gates, tokens)
    if workspace is None and _workspace_bytes(rows, seqlen, code):
        workspace = _workspace(rows, seqlen, code, tokens.device)
    if initial is not None:
        _check_state(initial, out, "initial")
        _launch(tokens.device, lib.ascan_forward_from, gates.data_ptr(), tokens.data_ptr(), initial.data_ptr(),
                out.data_ptr(), rows, seqlen, code, 1 if reverse else 0, _ptr(workspace),
                workspace.numel() if workspace is not None else 0)
    elif workspace is None:
        _launch(tokens.device, lib.ascan_forward, gates.data_ptr(), tokens.data_ptr(), out.data_ptr(), rows,
                seqlen, code, 1 if reverse else 0)
    else:
        _launch(tokens.device, lib.ascan_forward_split, gates.data_ptr(), tokens.data_ptr(), out.data_ptr(), rows,
                seqlen, code, 1 if reverse else 0, workspace.data_ptr(), workspace.numel())
    _after_split(workspace, "forward")


def backward(gates, states, grad_out, d_gates, d_tokens, workspace=None, initial=None, d_initial=None,
             reverse: bool = False) -> None:
    """Enqueue the fused backward scan on the current stream of the tensors' device.
    ``initial`` is the state the forward scan started from; ``d_initial``
    receives its gradient (left untouched for an empty sequence).  ``reverse``:
    the scan being differentiated ran backwards in time (``forward(..., reverse=True)``)."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gates, d_tokens)
    if workspace is None and _workspace_bytes(rows, seqlen, code):
        workspace = _workspace(rows, seqlen, code, gates.device)
    if reverse:
        _check_state(initial, states, "initial")
        _check_state(d_initial, states, "d_initial")
        _launch(gates.device, lib.ascan_backward_reverse, gates.data_ptr(), states.data_ptr(), _ptr(initial),
                grad_out.data_ptr(), d_gates.data_ptr(), d_tokens.data_ptr(), _ptr(d_initial), rows, seqlen, code,
                _ptr(workspace), workspace.numel() if workspace is not None else 0)
    elif initial is not None or d_initial is not None:
        _check_state(initial, states, "initial")
        _check_state(d_initial, states, "d_initial")
        _launch(gates.device, lib.ascan_backward_from, gates.data_ptr(), states.data_ptr(), _ptr(initial),
                grad_out.data_ptr(), d_gates.data_ptr(), d_tokens.data_ptr(), _ptr(d_initial), rows, seqlen, code,
                _ptr(workspace), workspace.numel() if workspace is not None else 0)
    elif workspace is None:
        _launch(gates.device, lib.ascan_backward, gates.data_ptr(), states.data_ptr(), grad_out.data_ptr(),
                d_gates.data_ptr(), d_tokens.data_ptr(), rows, seqlen, code)
    else:
        _launch(gates.device, lib.ascan_backward_split, gates.data_ptr(), states.data_ptr(), grad_out.data_ptr(),
                d_gates.data_ptr(), d_tokens.data_ptr(), rows, seqlen, code, workspace.data_ptr(), workspace.numel())
    _after_split(workspace, "backward")


def forward_gated(gate_inputs, tokens, out, gate: int, workspace=None, initial=None) -> None:
    """Forward scan whose gates are ``gate`` (an ascan_gate code) of ``gate_inputs``."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gate_inputs, tokens)
    if workspace is None:
        workspace = _workspace(rows, seqlen, code, tokens.device)
    _check_state(initial, out, "initial")
    _launch(tokens.device, lib.ascan_forward_gated, gate_inputs.data_ptr(), tokens.data_ptr(), _ptr(initial),
            out.data_ptr(), rows, seqlen, code, gate, _ptr(workspace),
            workspace.numel() if workspace is not None else 0)
    _after_split(workspace, "forward_gated")


def backward_gated(gate_inputs, states, grad_out, d_gate_inputs, d_tokens, gate: int, workspace=None,
                   initial=None, d_initial=None) -> None:
    """Backward of ``forward_gated``: gradients of the gate inputs, the tokens and the initial state."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gate_inputs, d_tokens)
    if workspace is None:
        workspace = _workspace(rows, seqlen, code, gate_inputs.device)
    _check_state(initial, states, "initial")
    _check_state(d_initial, states, "d_initial")
    _launch(gate_inputs.device, lib.ascan_backward_gated, gate_inputs.data_ptr(), states.data_ptr(), _ptr(initial),
            grad_out.data_ptr(), d_gate_inputs.data_ptr(), d_tokens.data_ptr(), _ptr(d_initial), rows, seqlen, code,
            gate, _ptr(workspace), workspace.numel() if workspace is not None else 0)
    _after_split(workspace, "backward_gated")


def backward_gated_values(gate_inputs, values, states, grad_out, d_gate_inputs, d_values, gate: int, workspace=None,
                          initial=None, d_initial=None) -> None:
    """Backward of ``forward_gated`` for a gate with values (``GATE_SIGMOID_LERP``:
    x[t] = a x[t-1] + (1 - a) values[t], a = sigmoid(gate_inputs); ``GATE_EXP_NORM``:
    x[t] = a x[t-1] + sqrt(1 - a^2) values[t], a = exp(gate_inputs)): gradients of the gate inputs,
    the values and the initial state."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gate_inputs, d_values)
    if workspace is None:
        workspace = _workspace(rows, seqlen, code, gate_inputs.device)
    _check_state(initial, states, "initial")
    _check_state(d_initial, states, "d_initial")
    _launch(gate_inputs.device, lib.ascan_backward_gated_values, gate_inputs.data_ptr(), values.data_ptr(),
            states.data_ptr(), _ptr(initial), grad_out.data_ptr(), d_gate_inputs.data_ptr(), d_values.data_ptr(),
            _ptr(d_initial), rows, seqlen, code, gate, _ptr(workspace),
            workspace.numel() if workspace is not None else 0)
    _after_split(workspace, "backward_gated_values")


def backward_lerp(gate_inputs, values, states, grad_out, d_gate_inputs, d_values, workspace=None,
                  initial=None, d_initial=None) -> None:
    """``backward_gated_values`` for the interpolating gate, through the library's ``ascan_backward_lerp``."""
    lib = _lib or load()
    rows, seqlen, code = _problem(gate_inputs, d_values)
    if workspace is None:
        workspace = _workspace(rows, seqlen, code, gate_inputs.device)
    _check_state(initial, states, "initial")
    _check_state(d_initial, states, "d_initial")
    _launch(gate_inputs.device, lib.ascan_backward_lerp, gate_inputs.data_ptr(), values.data_ptr(), states.data_ptr(),
            _ptr(initial), grad_out.data_ptr(), d_gate_inputs.data_ptr(), d_values.data_ptr(), _ptr(d_initial), rows,
            seqlen, code, _ptr(workspace), workspace.numel() if workspace is not None else 0)
    _after_split(workspace, "backward_lerp")


def workspace_timeouts(workspace) -> int:
    """Waits of a finished split call that ran out (synchronises the device)."""
    lib = _lib or load()
    header = workspace[:64].cpu().contiguous()
    return int(lib.ascan_workspace_timeouts(header.data_ptr()))
