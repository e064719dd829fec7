"""The HIP entry points as ``torch.library`` custom operators.

``torch.compile`` cannot trace a ctypes call; it can trace an opaque custom
operator that comes with a shape/dtype rule ("fake" implementation).  The
autograd nodes in ``warp``, ``scalar`` and ``complex`` therefore switch to
these operators while a graph is being captured and call the C ABI directly
otherwise (less Python overhead per call).  The reference advertises
``torch.compile`` for its torch scan only (README.md:36 of the reference).
"""

from typing import Tuple

import torch

from . import _abi


@torch.library.custom_op("accelerated_scan::scan_forward", mutates_args=())
def scan_forward(gates: torch.Tensor, tokens: torch.Tensor, reverse: bool) -> torch.Tensor:
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
    d_gates = torch.empty_like(gates)
    d_tokens = _empty_token_grad(gates, real_tokens)
    _abi.backward(gates, states, grad_out, d_gates, d_tokens)
    return d_gates, d_tokens


@scan_backward.register_fake
def _(gates, states, grad_out, real_tokens):
    return torch.empty_like(gates), _empty_token_grad(gates, real_tokens)


@torch.library.custom_op("accelerated_scan::scan_forward_from", mutates_args=())
def scan_forward_from(gates: torch.Tensor, tokens: torch.Tensor, initial: torch.Tensor, reverse: bool) -> torch.Tensor:
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
    d_gates = torch.empty_like(gates)
    d_tokens = _empty_token_grad(gates, real_tokens)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward(gates, states, grad_out, d_gates, d_tokens, initial=initial, d_initial=d_initial)
    return d_gates, d_tokens, d_initial


@scan_backward_from.register_fake
def _(gates, states, initial, grad_out, real_tokens):
    return torch.empty_like(gates), _empty_token_grad(gates, real_tokens), torch.empty_like(initial)


@torch.library.custom_op("accelerated_scan::scan_forward_gated", mutates_args=())
def scan_forward_gated(gate_inputs: torch.Tensor, tokens: torch.Tensor, initial: torch.Tensor, gate: int) -> torch.Tensor:
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
    d_gate_inputs = torch.empty_like(gate_inputs)
    d_tokens = torch.empty_like(gate_inputs)
    d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
    _abi.backward_gated(gate_inputs, states, grad_out, d_gate_inputs, d_tokens, gate, initial=initial,
                        d_initial=d_initial)
    return d_gate_inputs, d_tokens, d_initial


@scan_backward_gated.register_fake
def _(gate_inputs, states, initial, grad_out, gate):
    return torch.empty_like(gate_inputs), torch.empty_like(gate_inputs), torch.empty_like(initial)


def _empty_token_grad(gates: torch.Tensor, real_tokens: bool) -> torch.Tensor:
    """Token gradient buffer: real when complex gates were scanned over real tokens."""
    if real_tokens and gates.is_complex():
        return torch.empty(gates.shape, dtype=gates.real.dtype, device=gates.device)
    return torch.empty_like(gates)


def capturing() -> bool:
    """True while torch.compile is tracing the caller."""
    return torch.compiler.is_compiling()
