"""Any-length real scan with the argument names of accelerated_scan/scalar.py.

The reference implements this module with Triton kernels (scalar.py:16-86);
here it is the same HIP backend as ``warp``, which already accepts every
sequence length.  ``Scan`` saves ``(forget, states)`` and returns
``(d_forget, d_inputs)`` exactly as scalar.py:89-126 does.
"""

import torch

from . import _ops, warp


class Scan(torch.autograd.Function):
    @staticmethod
    def forward(ctx, forget, inputs):
        B, C, T = forget.shape
        assert inputs.shape == (B, C, T)
        assert forget.is_contiguous()
        assert inputs.is_contiguous()

        if _ops.capturing():
            states = _ops.scan_forward(forget, inputs, False)
        else:
            states = torch.empty_like(inputs)
            warp.warpscan_forward(forget, inputs, states, False)

        ctx.save_for_backward(forget, states)
        return states

    @staticmethod
    def backward(ctx, d_output):
        forget, states = ctx.saved_tensors

        d_output = d_output.contiguous()
        assert forget.is_contiguous()
        assert states.is_contiguous()

        if _ops.capturing():
            return _ops.scan_backward(forget, states, d_output, False)
        d_forget = torch.empty_like(forget)
        d_inputs = torch.empty_like(states)
        warp.warpscan_backward(forget, states, d_output, d_forget, d_inputs)
        return d_forget, d_inputs


def scan(forget, inputs, initial=None, reverse=False):
    """Solve ``x[t] = forget[t] * x[t-1] + inputs[t]`` for (B, C, T) tensors of any T.
    ``initial`` (shape (B, C), optional, not in the reference) is the state ``x[-1]``;
    ``reverse=True`` (not in the reference either) scans from the last element down,
    ``x[t] = forget[t] * x[t+1] + inputs[t]`` with ``x[T] = initial``, and is differentiable too."""
    if initial is not None or reverse:
        return warp.scan(forget, inputs, initial, reverse)
    return Scan.apply(forget, inputs)
