"""Scans whose gates come out of a non-linearity, with the non-linearity done inside the kernels.

``sigmoid_scan(gate_logits, tokens)`` equals
``warp.scan(torch.sigmoid(gate_logits), tokens)`` and is differentiable in the
logits, the tokens and the optional initial state, but never materialises the
gates: the forward kernel reads the logits and applies the sigmoid in
registers, the backward kernel writes the gradient of the logits directly.
Against the unfused pair of calls that saves the sigmoid's forward pass (one
read, one write), its backward pass (two reads, one write) and the saved gates
tensor.

``sigmoid_lerp_scan(gate_logits, values)`` solves the gated interpolation
``x[t] = a[t] * x[t-1] + (1 - a[t]) * values[t]`` with ``a = sigmoid(gate_logits)``
-- ``x[t] = torch.lerp(values[t], x[t-1], a[t])`` -- in which the tokens
``(1 - a) * values`` never exist in memory either: the forward kernel reads
logits and values (2 tensors in, 1 out, where the unfused sequence of sigmoid,
multiply and scan moves 9), the backward kernel reads logits, values, states
and the incoming gradient and writes both gradients (4 in, 2 out, against 21).

``exp_scan(log_gates, tokens)`` equals ``warp.scan(torch.exp(log_gates), tokens)``
the same way, for layers that keep their gates as logarithms (decay rates).  In
16-bit storage that is also the accurate way to hold gates close to 1:
bfloat16 has no value between 0.99609375 and 1, while a bfloat16 logarithm
of -0.001 carries three significant digits.

``exp_norm_scan(log_gates, values)`` solves
``x[t] = a[t] * x[t-1] + sqrt(1 - a[t]**2) * values[t]`` with ``a = exp(log_gates)``,
the update of RG-LRU / Hawk-style layers: the input scale keeps the variance of
the state at that of the values whatever the decay.  Gates, scales and scaled
tokens exist in registers only, and ``1 - a**2`` is evaluated without
cancellation for gates close to 1.

The reference's ``scan`` takes finished gates (accelerated_scan/warp.py:68-83);
the linear-RNN layers that call it (README.md:8,42 of the reference) typically
compute them with a sigmoid just before the scan.
"""

import torch

from . import _abi, _ops

_REAL_DTYPES = (torch.float32, torch.bfloat16, torch.float16)


def _check(gate_logits, tokens, initial):
    if gate_logits.dim() != 3 or tokens.shape != gate_logits.shape:
        raise RuntimeError("accelerated_scan: expected gate_logits and tokens of one shape (B, C, T)")
    if gate_logits.dtype not in _REAL_DTYPES or tokens.dtype != gate_logits.dtype:
        raise RuntimeError(
            f"accelerated_scan: unsupported tensor dtypes {gate_logits.dtype}, {tokens.dtype}: "
            "expecting gate_logits and tokens both bfloat16, float16 or float32"
        )
    if not (gate_logits.is_cuda and tokens.is_cuda and initial.is_cuda):
        raise RuntimeError("accelerated_scan: expected gate_logits, tokens and initial to be device tensors")
    if not (gate_logits.is_contiguous() and tokens.is_contiguous()):
        raise RuntimeError("accelerated_scan: expected gate_logits and tokens to be contiguous")
    if initial.shape != gate_logits.shape[:-1] or initial.dtype != gate_logits.dtype:
        raise RuntimeError(
            f"accelerated_scan: expected initial of shape {tuple(gate_logits.shape[:-1])} and dtype "
            f"{gate_logits.dtype}, got {tuple(initial.shape)} and {initial.dtype}"
        )


class GatedScan(torch.autograd.Function):
    """Autograd node of a scan with an in-kernel gate non-linearity (``gate``: an
    ascan_gate code other than the interpolating one): saves (gate_inputs, states,
    initial); no gates tensor exists."""

    @staticmethod
    def forward(ctx, gate_inputs, tokens, initial, gate):
        _check(gate_inputs, tokens, initial)
        initial = initial.contiguous()
        if _ops.capturing():
            states = _ops.scan_forward_gated(gate_inputs, tokens, initial, gate)
        else:
            states = torch.empty_like(gate_inputs)
            _abi.forward_gated(gate_inputs, tokens, states, gate, initial=initial)
        ctx.save_for_backward(gate_inputs, states, initial)
        ctx.gate = gate
        return states

    @staticmethod
    def backward(ctx, grad_output):
        gate_inputs, states, initial = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if _ops.capturing():
            return (*_ops.scan_backward_gated(gate_inputs, states, initial, grad_output, ctx.gate), None)
        d_gate_inputs = torch.empty_like(gate_inputs)
        d_tokens = torch.empty_like(gate_inputs)
        d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
        _abi.backward_gated(gate_inputs, states, grad_output, d_gate_inputs, d_tokens, ctx.gate,
                            initial=initial, d_initial=d_initial)
        return d_gate_inputs, d_tokens, d_initial, None


def sigmoid_scan(gate_logits, tokens, initial=None):
    """Solve ``x[t] = sigmoid(gate_logits[t]) * x[t-1] + tokens[t]``.

    Arguments:
        gate_logits (torch.Tensor): shape (B, C, T), contiguous; fp32, bf16 or fp16.
        tokens (torch.Tensor): shape (B, C, T), contiguous, same dtype.
        initial (torch.Tensor, optional): shape (B, C), the state ``x[-1]`` (zero if absent).

    Returns:
        (torch.Tensor): the states, shape (B, C, T).
    """
    if initial is None:
        initial = torch.zeros(gate_logits.shape[:-1], dtype=gate_logits.dtype, device=gate_logits.device)
    return GatedScan.apply(gate_logits, tokens, initial, _abi.GATE_SIGMOID)


def exp_scan(log_gates, tokens, initial=None):
    """Solve ``x[t] = exp(log_gates[t]) * x[t-1] + tokens[t]``.

    Arguments:
        log_gates (torch.Tensor): shape (B, C, T), contiguous; fp32, bf16 or fp16; logarithms of the gates.
        tokens (torch.Tensor): shape (B, C, T), contiguous, same dtype.
        initial (torch.Tensor, optional): shape (B, C), the state ``x[-1]`` (zero if absent).

    Returns:
        (torch.Tensor): the states, shape (B, C, T); differentiable in all arguments.
    """
    if initial is None:
        initial = torch.zeros(log_gates.shape[:-1], dtype=log_gates.dtype, device=log_gates.device)
    return GatedScan.apply(log_gates, tokens, initial, _abi.GATE_EXP)


class ValuesScan(torch.autograd.Function):
    """Autograd node of the scans whose second input holds values (``gate``: the interpolating
    or the normalised exponential ascan_gate code): saves (gate_inputs, values, states, initial)."""

    @staticmethod
    def forward(ctx, gate_inputs, values, initial, gate):
        _check(gate_inputs, values, initial)
        initial = initial.contiguous()
        if _ops.capturing():
            states = _ops.scan_forward_gated(gate_inputs, values, initial, gate)
        else:
            states = torch.empty_like(gate_inputs)
            _abi.forward_gated(gate_inputs, values, states, gate, initial=initial)
        ctx.save_for_backward(gate_inputs, values, states, initial)
        ctx.gate = gate
        return states

    @staticmethod
    def backward(ctx, grad_output):
        gate_inputs, values, states, initial = ctx.saved_tensors
        grad_output = grad_output.contiguous()
        if _ops.capturing():
            return (*_ops.scan_backward_gated_values(gate_inputs, values, states, initial, grad_output, ctx.gate), None)
        d_gate_inputs = torch.empty_like(gate_inputs)
        d_values = torch.empty_like(gate_inputs)
        d_initial = torch.zeros_like(initial)  # stays zero for an empty sequence
        _abi.backward_gated_values(gate_inputs, values, states, grad_output, d_gate_inputs, d_values, ctx.gate,
                                   initial=initial, d_initial=d_initial)
        return d_gate_inputs, d_values, d_initial, None


def sigmoid_lerp_scan(gate_logits, values, initial=None):
    """Solve ``x[t] = a[t] * x[t-1] + (1 - a[t]) * values[t]`` with ``a = sigmoid(gate_logits)``.

    Arguments:
        gate_logits (torch.Tensor): shape (B, C, T), contiguous; fp32, bf16 or fp16.
        values (torch.Tensor): shape (B, C, T), contiguous, same dtype.
        initial (torch.Tensor, optional): shape (B, C), the state ``x[-1]`` (zero if absent).

    Returns:
        (torch.Tensor): the states, shape (B, C, T); differentiable in all arguments.
    """
    if initial is None:
        initial = torch.zeros(gate_logits.shape[:-1], dtype=gate_logits.dtype, device=gate_logits.device)
    return ValuesScan.apply(gate_logits, values, initial, _abi.GATE_SIGMOID_LERP)


def exp_norm_scan(log_gates, values, initial=None):
    """Solve ``x[t] = a[t] * x[t-1] + sqrt(1 - a[t]**2) * values[t]`` with ``a = exp(log_gates)``.

    Arguments:
        log_gates (torch.Tensor): shape (B, C, T), contiguous; fp32, bf16 or fp16; logarithms of the
            gates, negative (at 0 the input scale vanishes and its derivative is unbounded; the backward pass
            takes that derivative as 0 there, so a stored 0 gives finite gradients).
        values (torch.Tensor): shape (B, C, T), contiguous, same dtype.
        initial (torch.Tensor, optional): shape (B, C), the state ``x[-1]`` (zero if absent).

    Returns:
        (torch.Tensor): the states, shape (B, C, T); differentiable in all arguments.
    """
    if initial is None:
        initial = torch.zeros(log_gates.shape[:-1], dtype=log_gates.dtype, device=log_gates.device)
    return ValuesScan.apply(log_gates, values, initial, _abi.GATE_EXP_NORM)
