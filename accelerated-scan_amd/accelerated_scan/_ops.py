"""The HIP entry points as ``torch.library`` custom operators.

``torch.compile`` cannot trace a ctypes call; it can trace an opaque custom
operator that comes with a shape/dtype rule ("fake" implementation).  The
autograd nodes in ``warp``, ``scalar`` and ``complex`` therefore switch to
these operators while a graph is being captured and call the C ABI directly
otherwise (less Python overhead per call).  The reference advertises
``torch.compile`` for its torch scan only (README.md:36 of the reference).

The three forward operators carry autograd formulas of their own
(``torch.library.register_autograd``, at the end of this file), so
``torch.ops.accelerated_scan.scan_forward(gates, tokens, False)`` is
differentiable without any ``autograd.Function`` around it, in eager mode and
under ``torch.compile``.  Every operator validates its arguments itself: they
are public as ``torch.ops.accelerated_scan.*``.
"""

from typing import Tuple

import torch

from . import _abi


def _check_dense(first: torch.Tensor, others, token_like=None, states=()) -> None:
    """All tensors of a call: device tensors on one device, contiguous, of one
    shape; ``others`` share the dtype of ``first``; ``token_like`` may be
    float32 beside complex64; ``states`` hold one element per row."""
    def fail(what):
        raise RuntimeError(f"accelerated_scan: expected {what}")

    if not first.is_cuda:
        fail("device tensors")
    if first.dim() < 1:
        fail("tensors with a sequence axis")
    for t in tuple(others) + ((token_like,) if token_like is not None else ()):
        if not t.is_cuda or t.device != first.device:
            fail("all tensors on one GPU")
        if t.shape != first.shape:
            fail(f"tensors of one shape, got {tuple(first.shape)} and {tuple(t.shape)}")
        if not t.is_contiguous():
            fail("contiguous tensors")
    if not first.is_contiguous():
        fail("contiguous tensors")
    for t in others:
        if t.dtype != first.dtype:
            fail(f"tensors of one dtype, got {first.dtype} and {t.dtype}")
    if token_like is not None:
        _abi.dtype_code(first.dtype, token_like.dtype)  # raises for unsupported combinations
    for t in states:
        if (not t.is_cuda or t.device != first.device or t.dtype != first.dtype
                or t.shape != first.shape[:-1] or not t.is_contiguous()):
            fail(f"a contiguous {first.dtype} state of shape {tuple(first.shape[:-1])} on {first.device}")


@torch.library.custom_op("accelerated_scan::scan_forward", mutates_args=())
def scan_forward(gates: torch.Tensor, tokens: torch.Tensor, reverse: bool) -> torch.Tensor:
    _check_dense(gates, (), token_like=tokens)
    out = torch.empty_like(gates)  # complex gates with real tokens give complex states
    _abi.forward(gates, tokens, out, reverse)
    return out


@scan_forward.register_fake
def _(gates, tokens, reverse):
    return torch.empty_like(gates)


@torch.library.custom_op("accelerated_scan::scan_backward", mutates_args=())
def scan_backward(
    gates: torch.Tensor, states: torch.Tensor, grad_out: torch.Tensor, real_tokens: bool
) -> Tuple[torch.Tensor, torch.Tensor]:
    _check_dense(gates, (states, grad_out))
    d_gates = torch.empty_like(gates)
    d_tokens = _empty_token_grad(gates, real_tokens)
    _abi.backward(gates, states, grad_out, d_gates, d_tokens)
    return d_gates, d_tokens


@scan_backward.register_fake
def _(gates, states, grad_out, real_tokens):
    return torch.empty_like(gates), _empty_token_grad(gates, real_tokens)


@torch.library.custom_op("accelerated_scan::scan_forward_from", mutates_args=())
def scan_forward_from(gates: torch.Tensor, tokens: torch.Tensor, initial: torch.Tensor, reverse: bool) -> torch.Tensor:
    _check_dense(gates, (), token_like=tokens, states=(initial,))
    out = torch.empty_like(gates)
    _abi.forward(gates, tokens, out, reverse, initial=initial)
    return out


@scan_forward_from.register_fake
def _(gates, tokens, initial, reverse):
    return torch.empty_like(gates)


@torch.library.custom_op("accelerated_scan::scan_backward_from", mutates_args=())
def scan_backward_from(
    gates: torch.Tensor, states: torch.Tensor, initial: torch.Tensor, grad_out: torch.Tensor, real_tokens: bool
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_dense(gates, (states, grad_out), states=(initial,))
    d_gates = torch.empty_like(gates)
    d_tokens = _empty_token_grad(gates, real_tokens)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward(gates, states, grad_out, d_gates, d_tokens, initial=initial, d_initial=d_initial)
    return d_gates, d_tokens, d_initial


@scan_backward_from.register_fake
def _(gates, states, initial, grad_out, real_tokens):
    return torch.empty_like(gates), _empty_token_grad(gates, real_tokens), torch.empty_like(initial)


@torch.library.custom_op("accelerated_scan::scan_backward_reverse", mutates_args=())
def scan_backward_reverse(
    gates: torch.Tensor, states: torch.Tensor, initial: torch.Tensor, grad_out: torch.Tensor, real_tokens: bool
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """Backward pass of a reverse scan (``scan_forward`` / ``scan_forward_from`` with ``reverse=True``)."""
    _check_dense(gates, (states, grad_out), states=(initial,))
    d_gates = torch.empty_like(gates)
    d_tokens = _empty_token_grad(gates, real_tokens)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward(gates, states, grad_out, d_gates, d_tokens, initial=initial, d_initial=d_initial, reverse=True)
    return d_gates, d_tokens, d_initial


@scan_backward_reverse.register_fake
def _(gates, states, initial, grad_out, real_tokens):
    return torch.empty_like(gates), _empty_token_grad(gates, real_tokens), torch.empty_like(initial)


@torch.library.custom_op("accelerated_scan::scan_forward_gated", mutates_args=())
def scan_forward_gated(gate_inputs: torch.Tensor, tokens: torch.Tensor, initial: torch.Tensor, gate: int) -> torch.Tensor:
    _check_dense(gate_inputs, (tokens,), states=(initial,))
    out = torch.empty_like(gate_inputs)
    _abi.forward_gated(gate_inputs, tokens, out, gate, initial=initial)
    return out


@scan_forward_gated.register_fake
def _(gate_inputs, tokens, initial, gate):
    return torch.empty_like(gate_inputs)


@torch.library.custom_op("accelerated_scan::scan_backward_gated", mutates_args=())
def scan_backward_gated(
    gate_inputs: torch.Tensor, states: torch.Tensor, initial: torch.Tensor, grad_out: torch.Tensor, gate: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_dense(gate_inputs, (states, grad_out), states=(initial,))
    d_gate_inputs = torch.empty_like(gate_inputs)
    d_tokens = torch.empty_like(gate_inputs)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward_gated(gate_inputs, states, grad_out, d_gate_inputs, d_tokens, gate, initial=initial,
                        d_initial=d_initial)
    return d_gate_inputs, d_tokens, d_initial


@scan_backward_gated.register_fake
def _(gate_inputs, states, initial, grad_out, gate):
    return torch.empty_like(gate_inputs), torch.empty_like(gate_inputs), torch.empty_like(initial)


@torch.library.custom_op("accelerated_scan::scan_backward_lerp", mutates_args=())
def scan_backward_lerp(
    gate_inputs: torch.Tensor, values: torch.Tensor, states: torch.Tensor, initial: torch.Tensor, grad_out: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_dense(gate_inputs, (values, states, grad_out), states=(initial,))
    d_gate_inputs = torch.empty_like(gate_inputs)
    d_values = torch.empty_like(gate_inputs)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward_lerp(gate_inputs, values, states, grad_out, d_gate_inputs, d_values, initial=initial,
                       d_initial=d_initial)
    return d_gate_inputs, d_values, d_initial


@scan_backward_lerp.register_fake
def _(gate_inputs, values, states, initial, grad_out):
    return torch.empty_like(gate_inputs), torch.empty_like(gate_inputs), torch.empty_like(initial)


@torch.library.custom_op("accelerated_scan::scan_backward_gated_values", mutates_args=())
def scan_backward_gated_values(
    gate_inputs: torch.Tensor, values: torch.Tensor, states: torch.Tensor, initial: torch.Tensor,
    grad_out: torch.Tensor, gate: int
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    _check_dense(gate_inputs, (values, states, grad_out), states=(initial,))
    d_gate_inputs = torch.empty_like(gate_inputs)
    d_values = torch.empty_like(gate_inputs)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward_gated_values(gate_inputs, values, states, grad_out, d_gate_inputs, d_values, gate, initial=initial,
                               d_initial=d_initial)
    return d_gate_inputs, d_values, d_initial


@scan_backward_gated_values.register_fake
def _(gate_inputs, values, states, initial, grad_out, gate):
    return torch.empty_like(gate_inputs), torch.empty_like(gate_inputs), torch.empty_like(initial)


def _empty_token_grad(gates: torch.Tensor, real_tokens: bool) -> torch.Tensor:
    """Token gradient buffer: real when complex gates were scanned over real tokens."""
    if real_tokens and gates.is_complex():
        return torch.empty(gates.shape, dtype=gates.real.dtype, device=gates.device)
    return torch.empty_like(gates)


def capturing() -> bool:
    """True while torch.compile is tracing the caller."""
    return torch.compiler.is_compiling()


# ---------------------------------------------------------------------------
# Autograd formulas of the forward operators.  The gradient of a scan is the
# fused backward operator (accelerated_scan/warp.py:50-65 of the reference:
# g[t] = grad[t] + gates[t+1] * g[t+1], d_tokens = g, d_gates[t] = g[t] * x[t-1]).
# A reverse scan has a fused backward operator of its own, the mirror image in time.
# ---------------------------------------------------------------------------
def _real_tokens(gates: torch.Tensor, tokens: torch.Tensor) -> bool:
    return gates.is_complex() and not tokens.is_complex()


def _setup_scan_forward(ctx, inputs, output):
    gates, tokens, reverse = inputs
    ctx.save_for_backward(gates, output)
    ctx.reverse = reverse
    ctx.real_tokens = _real_tokens(gates, tokens)


def _backward_scan_forward(ctx, grad):
    gates, states = ctx.saved_tensors
    grad = grad.contiguous()
    if ctx.reverse:
        zero = torch.zeros(gates.shape[:-1], dtype=gates.dtype, device=gates.device)
        d_gates, d_tokens, _ = scan_backward_reverse(gates, states, zero, grad, ctx.real_tokens)
        return d_gates, d_tokens, None
    d_gates, d_tokens = scan_backward(gates, states, grad, ctx.real_tokens)
    return d_gates, d_tokens, None


torch.library.register_autograd(
    "accelerated_scan::scan_forward", _backward_scan_forward, setup_context=_setup_scan_forward)


def _setup_scan_forward_from(ctx, inputs, output):
    gates, tokens, initial, reverse = inputs
    ctx.save_for_backward(gates, output, initial)
    ctx.reverse = reverse
    ctx.real_tokens = _real_tokens(gates, tokens)


def _backward_scan_forward_from(ctx, grad):
    gates, states, initial = ctx.saved_tensors
    grad = grad.contiguous()
    if ctx.reverse:
        d_gates, d_tokens, d_initial = scan_backward_reverse(gates, states, initial, grad, ctx.real_tokens)
        return d_gates, d_tokens, d_initial, None
    d_gates, d_tokens, d_initial = scan_backward_from(gates, states, initial, grad, ctx.real_tokens)
    return d_gates, d_tokens, d_initial, None


torch.library.register_autograd(
    "accelerated_scan::scan_forward_from", _backward_scan_forward_from, setup_context=_setup_scan_forward_from)


def _setup_scan_forward_gated(ctx, inputs, output):
    gate_inputs, tokens, initial, gate = inputs
    if gate in _abi.GATES_WITH_VALUES:  # the second input holds values, and the backward pass reads them
        ctx.save_for_backward(gate_inputs, output, initial, tokens)
    else:
        ctx.save_for_backward(gate_inputs, output, initial)
    ctx.gate = gate


def _backward_scan_forward_gated(ctx, grad):
    if ctx.gate in _abi.GATES_WITH_VALUES:
        gate_inputs, states, initial, values = ctx.saved_tensors
        d_gate_inputs, d_values, d_initial = scan_backward_gated_values(gate_inputs, values, states, initial,
                                                                        grad.contiguous(), ctx.gate)
        return d_gate_inputs, d_values, d_initial, None
    gate_inputs, states, initial = ctx.saved_tensors
    d_gate_inputs, d_tokens, d_initial = scan_backward_gated(gate_inputs, states, initial, grad.contiguous(), ctx.gate)
    return d_gate_inputs, d_tokens, d_initial, None


torch.library.register_autograd(
    "accelerated_scan::scan_forward_gated", _backward_scan_forward_gated, setup_context=_setup_scan_forward_gated)
