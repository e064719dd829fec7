"""Real-valued scan on the HIP backend.

Public names and semantics follow accelerated_scan/warp.py:29-83 of the
reference: ``warpscan_forward``, ``warpscan_backward``, ``scan_forward``,
``Scan`` and ``scan``.  Differences, all supersets: any sequence length
T >= 1 (the reference accepts 12 powers of two, warp.cuh:282-380), 64-bit
offsets, fp32 accumulation for bf16 / fp16 storage, and no zero-fill of the
output before the kernel runs.
"""

import torch

from . import _abi, _ops, stateful

_REAL_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


def _require(cond: bool, what: str) -> None:
    # the reference reports these through TORCH_CHECK, which raises RuntimeError
    if not cond:
        raise RuntimeError(f"accelerated_scan: expected {what}")


def _check_dtype(t: torch.Tensor) -> None:
    if t.dtype not in _REAL_DTYPES:
        raise RuntimeError(
            f"accelerated_scan: unsupported tensor dtype {t.dtype}: expecting bfloat16, float16 or float32"
        )


def _check_launch(tensors, names) -> None:
    """Device, layout, dtype and shape checks shared by the two launchers; the
    first tensor is the yardstick.  The passing case builds no message."""
    first = tensors[0]
    dtype, shape, device = first.dtype, first.shape, first.device
    for t in tensors:
        if not (t.is_cuda and t.dtype == dtype and t.shape == shape and t.device == device and t.is_contiguous()):
            break
    else:
        if dtype in _REAL_DTYPES:
            return
    for t, name in zip(tensors, names):
        _require(t.is_cuda, f"{name} to be a device tensor")
        _require(t.is_contiguous(), f"{name} to be contiguous")
        _require(t.dtype == dtype, f"{name} to have the dtype of {names[0]}")
        _require(t.shape == shape, f"{name} to have the shape of {names[0]}")
        _require(t.device == device, f"{name} to be on the device of {names[0]}")
    _check_dtype(first)


def warpscan_forward(gates, tokens, out, reverse=False):
    """Write the scan of (gates, tokens) into ``out`` and return ``out``.

    Checks mirror accelerated_scan/warp.cuh:394-405: device tensors,
    contiguous inputs, one dtype for all three.  ``reverse=True`` solves
    ``y[t] = gates[t] * y[t+1] + tokens[t]``.
    """
    _check_launch((tokens, gates, out), ("tokens", "gates", "out"))
    _abi.forward(gates, tokens, out, reverse)
    return out


def warpscan_backward(gates, output, outGrad, gateGradOut, tokenGradOut):
    """Fused backward: fills ``gateGradOut`` and ``tokenGradOut``.

    ``output`` is the forward result, ``outGrad`` the incoming gradient.
    Checks mirror accelerated_scan/warp.cuh:407-421.
    """
    _check_launch((gates, output, outGrad, gateGradOut, tokenGradOut),
                  ("gates", "output", "outGrad", "gateGradOut", "tokenGradOut"))
    _abi.backward(gates, output, outGrad, gateGradOut, tokenGradOut)


def scan_forward(gates, tokens, reverse=False):
    """Forward (or reverse) scan without autograd (accelerated_scan/warp.py:32-35)."""
    if _ops.capturing():
        return _ops.scan_forward(gates, tokens, reverse)
    output = torch.empty_like(tokens)
    warpscan_forward(gates, tokens, output, reverse)
    return output


class Scan(torch.autograd.Function):
    """Autograd node of the scan (accelerated_scan/warp.py:38-65)."""

    @staticmethod
    def forward(ctx, gates, tokens):
        B, C, T = gates.shape
        assert tokens.shape == (B, C, T)
        assert gates.is_contiguous()
        assert tokens.is_contiguous()

        states = scan_forward(gates, tokens)
        ctx.save_for_backward(states, gates)
        return states

    @staticmethod
    def backward(ctx, grad_output):
        # g[t] = grad_output[t] + gates[t+1] * g[t+1]; d_tokens = g; d_gates[t] = g[t] * states[t-1]
        states, gates = ctx.saved_tensors

        grad_output = grad_output.contiguous()
        assert states.is_contiguous()
        assert gates.is_contiguous()

        if _ops.capturing():
            return _ops.scan_backward(gates, states, grad_output, False)
        d_gates = torch.empty_like(gates)
        d_tokens = torch.empty_like(gates)
        warpscan_backward(gates, states, grad_output, d_gates, d_tokens)
        return d_gates, d_tokens


def scan(gates, tokens, initial=None, reverse=False):
    """Solve the first-order recurrence ``x[t] = gates[t] * x[t-1] + tokens[t]``.

    Arguments:
        gates (torch.Tensor): shape (B, C, T), contiguous, on the GPU.
        tokens (torch.Tensor): shape (B, C, T), contiguous, same dtype.
        initial (torch.Tensor, optional): shape (B, C), the state ``x[-1]`` to
            start from (not in the reference, which starts from zero).
        reverse (bool, optional): solve ``x[t] = gates[t] * x[t+1] + tokens[t]`` from the
            last element down instead (``initial`` is then ``x[T]``); differentiable like
            the forward scan (not in the reference, whose reverse scan has no gradient).

    Returns:
        (torch.Tensor): shape (B, C, T), the states ``x``; differentiable in
        all arguments.
    """
    if initial is not None or reverse:
        _check_dtype(gates)
        return stateful.scan(gates, tokens, initial, reverse)
    return Scan.apply(gates, tokens)
