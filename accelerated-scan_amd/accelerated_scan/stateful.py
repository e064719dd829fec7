"""Scans that start from a given state, for sequences processed in chunks.

``scan(gates, tokens, initial)`` solves ``x[t] = gates[t] * x[t-1] + tokens[t]``
with ``x[-1] = initial`` (one state per (batch, channel) pair) and is
differentiable in all three arguments.  The last state of a chunk,
``states[..., -1]``, is the ``initial`` of the next one: streaming inference
keeps only that (B, C) tensor between calls, and truncated back-propagation
through time can let gradients flow across the chunk boundary through it.

The reference has no such entry point: its scans start from zero
(accelerated_scan/warp.cuh:76, scalar.py:28, complex.py:32-33).  The
``scan`` functions of ``warp``, ``scalar`` and ``complex`` accept
``initial=`` as an optional keyword and end up here; without it they behave
exactly as the reference's.
"""

import torch

from . import _abi, _ops


def _check(gates, tokens, initial):
    if gates.dim() != 3 or tokens.shape != gates.shape:
        raise RuntimeError("accelerated_scan: expected gates and tokens of one shape (B, C, T)")
    if not (gates.is_cuda and tokens.is_cuda and initial.is_cuda):
        raise RuntimeError("accelerated_scan: expected gates, tokens and initial to be device tensors")
    if not (gates.is_contiguous() and tokens.is_contiguous()):
        raise RuntimeError("accelerated_scan: expected gates and tokens to be contiguous")
    if initial.shape != gates.shape[:-1] or initial.dtype != gates.dtype:
        raise RuntimeError(
            f"accelerated_scan: expected initial of shape {tuple(gates.shape[:-1])} and dtype {gates.dtype}, "
            f"got {tuple(initial.shape)} and {initial.dtype}"
        )
    _abi.dtype_code(gates.dtype, tokens.dtype)  # raises for unsupported combinations


def scan_forward(gates, tokens, initial, reverse=False):
    """States of the scan started from ``initial``, without autograd.
    ``reverse=True`` solves ``y[t] = gates[t] * y[t+1] + tokens[t]`` with ``y[T] = initial``."""
    _check(gates, tokens, initial)
    initial = initial.contiguous()
    if _ops.capturing():
        return _ops.scan_forward_from(gates, tokens, initial, reverse)
    out = torch.empty_like(gates)
    _abi.forward(gates, tokens, out, reverse, initial=initial)
    return out


class Scan(torch.autograd.Function):
    """Autograd node: saves (gates, states, initial), returns (d_gates, d_tokens, d_initial)."""

    @staticmethod
    def forward(ctx, gates, tokens, initial, reverse=False):
        initial = initial.contiguous()
        states = scan_forward(gates, tokens, initial, reverse)
        ctx.save_for_backward(gates, states, initial)
        ctx.real_tokens = gates.is_complex() and not tokens.is_complex()
        ctx.reverse = reverse
        return states

    @staticmethod
    def backward(ctx, grad_output):
        gates, states, initial = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if _ops.capturing():
            op = _ops.scan_backward_reverse if ctx.reverse else _ops.scan_backward_from
            return (*op(gates, states, initial, grad_output, ctx.real_tokens), None)
        d_gates = torch.empty_like(gates)
        if ctx.real_tokens:
            d_tokens = torch.empty(gates.shape, dtype=gates.real.dtype, device=gates.device)
        else:
            d_tokens = torch.empty_like(gates)
        d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
        _abi.backward(gates, states, grad_output, d_gates, d_tokens, initial=initial, d_initial=d_initial,
                      reverse=ctx.reverse)
        return d_gates, d_tokens, d_initial, None


def scan(gates, tokens, initial=None, reverse=False):
    """Solve ``x[t] = gates[t] * x[t-1] + tokens[t]`` from ``x[-1] = initial``, or with
    ``reverse=True`` ``y[t] = gates[t] * y[t+1] + tokens[t]`` from ``y[T] = initial``.

    Arguments:
        gates (torch.Tensor): shape (B, C, T), contiguous; fp32, bf16, fp16 or complex64.
        tokens (torch.Tensor): shape (B, C, T), contiguous, the dtype of gates
            (or float32 with complex64 gates).
        initial (torch.Tensor, optional): shape (B, C), the dtype of gates; zeros if absent.
        reverse (bool): scan from the last element to the first.  The reference's reverse
            scan (accelerated_scan/warp.py:32-35) is not differentiable; this one is, through
            a fused backward kernel of its own, so a sequence can be scanned in both directions.

    Returns:
        (torch.Tensor): states of shape (B, C, T), differentiable in gates, tokens and
        initial; ``states[..., -1]`` (``states[..., 0]`` for a reverse scan) is the state
        to hand to the next chunk.
    """
    if initial is None:
        initial = torch.zeros(gates.shape[:-1], dtype=gates.dtype, device=gates.device)
    return Scan.apply(gates, tokens, initial, reverse)
