"""Complex64 scan on the HIP backend (operator of accelerated_scan/complex.py:157-239).

``forget`` must be complex; ``inputs`` may be complex or real (a real tensor
is read as having zero imaginary part and receives a real gradient).  The
backward pass follows complex.py:79-92: with g the adjoint of the states,
``g[t] = d_output[t] + conj(forget[t+1]) * g[t+1]``, ``d_inputs = g`` and
``d_forget[t] = g[t] * conj(states[t-1])``.
"""

import torch

from . import _abi, _ops, stateful


def _require(cond: bool, what: str) -> None:
    if not cond:
        raise RuntimeError(f"accelerated_scan: expected {what}")


def _launch_forward(forget, inputs, states):
    for t, name in ((forget, "forget"), (inputs, "inputs"), (states, "states")):
        _require(t.is_cuda, f"{name} to be a device tensor")
        _require(t.device == forget.device, f"{name} to be on the device of forget")
    _require(forget.dtype == torch.complex64 and states.dtype == torch.complex64, "forget and states to be complex64")
    _require(inputs.dtype in (torch.complex64, torch.float32), "inputs to be complex64 or float32")
    _abi.forward(forget, inputs, states, False)


def _launch_backward(forget, states, d_output, d_forget, d_inputs):
    for t, name in ((forget, "forget"), (states, "states"), (d_output, "d_output"), (d_forget, "d_forget")):
        _require(t.is_cuda, f"{name} to be a device tensor")
        _require(t.dtype == torch.complex64, f"{name} to be complex64")
        _require(t.shape == forget.shape, f"{name} to have the shape of forget")
        _require(t.device == forget.device, f"{name} to be on the device of forget")
    _require(d_inputs.dtype in (torch.complex64, torch.float32), "d_inputs to be complex64 or float32")
    _abi.backward(forget, states, d_output, d_forget, d_inputs)


class Scan(torch.autograd.Function):
    @staticmethod
    def forward(ctx, forget, inputs):
        if not torch.is_complex(forget):
            raise TypeError("forget must be a complex tensor")
        real_inputs = not torch.is_complex(inputs)
        B, C, T = forget.shape
        assert inputs.shape == (B, C, T)
        assert forget.is_contiguous()
        assert inputs.is_contiguous()

        # Real inputs are not promoted to a complex copy (the reference does,
        # complex.py:168-169): the kernel reads them as (input, 0).
        if _ops.capturing():
            states = _ops.scan_forward(forget, inputs, False)
        else:
            states = torch.empty_like(forget)
            _launch_forward(forget, inputs, states)

        ctx.save_for_backward(forget, states)
        ctx.real_inputs = real_inputs
        return states

    @staticmethod
    def backward(ctx, d_output):
        forget, states = ctx.saved_tensors

        d_output = d_output.contiguous()
        assert forget.is_contiguous()
        assert states.is_contiguous()

        # For real inputs the kernel writes only the real part of the input
        # gradient (what complex.py:217-218 keeps).
        if _ops.capturing():
            d_forget, d_inputs = _ops.scan_backward(forget, states, d_output, ctx.real_inputs)
        else:
            d_forget = torch.empty_like(forget)
            if ctx.real_inputs:
                d_inputs = torch.empty(forget.shape, dtype=torch.float32, device=forget.device)
            else:
                d_inputs = torch.empty_like(states)
            _launch_backward(forget, states, d_output, d_forget, d_inputs)
        return d_forget, d_inputs


def scan(forget, inputs, initial=None, reverse=False):
    """Solve ``x[t] = forget[t] * x[t-1] + inputs[t]`` over complex numbers.

    Arguments:
        forget (torch.Tensor): shape (B, C, T), complex64, contiguous.
        inputs (torch.Tensor): shape (B, C, T), complex64 or float32, contiguous.
        initial (torch.Tensor, optional): shape (B, C), complex64, the state
            ``x[-1]`` to start from (not in the reference, which starts from zero).
        reverse (bool, optional): solve ``x[t] = forget[t] * x[t+1] + inputs[t]`` from the
            last element down (``initial`` is then ``x[T]``); differentiable like the
            forward scan (not in the reference).

    Returns:
        (torch.Tensor): complex64 states of shape (B, C, T).
    """
    if initial is not None or reverse:
        if not torch.is_complex(forget):
            raise TypeError("forget must be a complex tensor")
        return stateful.scan(forget, inputs, initial, reverse)
    return Scan.apply(forget, inputs)
