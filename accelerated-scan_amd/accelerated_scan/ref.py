"""``accelerated_scan.ref`` by name, on the HIP backend.

The reference ships a pure-torch tree scan under this name
(accelerated_scan/ref.py:49-87) as the third interchangeable import beside
``warp`` and ``scalar`` (README.md:25-27 of the reference), with a
``reverse`` flag and gradients through autograd.  This module keeps the import
and the signature working for code written against it, but it is not a second
implementation: ``scan`` runs the same HIP kernels as ``warp.scan`` /
``complex.scan`` -- forward or reverse in time, differentiable either way --
so it needs device tensors and one of the library's dtypes.  There is no CPU
path here: host tensors are refused like everywhere else in the package.

What differs from the reference's function, therefore:
  * the arithmetic hooks (``mul``, ``add``, ``zeros_like``, ``ones_like``)
    exist in the signature but only their defaults are accepted -- the kernels
    compute ``gates * x + tokens`` in fp32 (complex64: in complex fp32);
  * results agree with the tree scan to rounding (sequential fused arithmetic
    instead of log2(T) levels), not bit for bit;
  * dtypes: float32, bfloat16, float16, complex64 (the tree scan takes
    anything torch can multiply).

``split`` and ``merge`` (ref.py:8-46), the two views the tree scan is made of,
are provided as well; they are plain tensor reshapes on any device.
"""

import torch

from . import stateful, warp
from . import complex as _complex


def split(x: torch.Tensor):
    """Even-indexed and odd-indexed elements of the last axis: (B, C, T) -> two (B, C, T//2) views.

    >>> split(torch.tensor([1,2,3,4,5,6,7,8])[None, None, :])
    (tensor([[[1, 3, 5, 7]]]), tensor([[[2, 4, 6, 8]]]))
    """
    pairs = x.unflatten(-1, (x.shape[-1] // 2, 2))
    return pairs.select(-1, 0), pairs.select(-1, 1)


def merge(lefts: torch.Tensor, rights: torch.Tensor) -> torch.Tensor:
    """Inverse of ``split``: interleaves two (B, C, T//2) tensors into one (B, C, T).

    >>> merge(torch.tensor([1,3,5,7])[None, None, :], torch.tensor([2,4,6,8])[None, None, :])
    tensor([[[1, 2, 3, 4, 5, 6, 7, 8]]])
    """
    return torch.stack((lefts, rights), dim=-1).flatten(-2)


def scan(gates, tokens, mul=torch.mul, add=torch.add, zeros_like=torch.zeros_like, ones_like=torch.ones_like,
         reverse=False):
    """Solve ``x[t] = gates[t] * x[t-1] + tokens[t]`` (``reverse=True``:
    ``x[t] = gates[t] * x[t+1] + tokens[t]`` from the last element down).

    Arguments:
        gates (torch.Tensor): shape (B, C, T), contiguous, on the GPU; float32,
            bfloat16, float16 or complex64.
        tokens (torch.Tensor): shape (B, C, T), contiguous, same dtype (float32
            is also accepted with complex64 gates).
        mul, add, zeros_like, ones_like: the reference's arithmetic hooks; only
            the torch defaults are supported.
        reverse (bool): scan direction.

    Returns:
        (torch.Tensor): shape (B, C, T), differentiable in gates and tokens.
    """
    if mul is not torch.mul or add is not torch.add or zeros_like is not torch.zeros_like \
            or ones_like is not torch.ones_like:
        raise NotImplementedError(
            "accelerated_scan.ref.scan runs compiled kernels: custom mul / add / zeros_like / ones_like "
            "are not supported"
        )
    if not (gates.is_cuda and tokens.is_cuda):
        raise RuntimeError("accelerated_scan: expected gates and tokens to be device tensors (there is no CPU path)")
    if reverse:
        return stateful.scan(gates, tokens, None, True)
    if torch.is_complex(gates):
        return _complex.scan(gates, tokens)
    return warp.scan(gates, tokens)
