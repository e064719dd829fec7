"""ORACLE (test infrastructure, not part of the product).

CPU restatement in plain torch of the reference's tree scan,
``accelerated_scan/ref.py:49-121``: the operator every test of the reference
compares against (tests/test_eq.py:26-62, tests/tests_eq_complex.py:55-86).
Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; nothing under ``accelerated-scan_amd/``
does.

The reference recurses (``scan1`` calls itself once per tree level); this
restatement runs the same levels as two loops, an up-sweep that keeps each
level's near children and a down-sweep that consumes them, issuing the same
``mul`` / ``add`` calls with the same operands in the same order, so fp32
results are bit-identical to the reference's.  That claim is pinned by the
fixtures in tests/golden/ (written from the reference itself); values are
pinned independently by the sequential fp64 recurrence in oracle/seqscan.c and
by closed forms (cumsum / cumprod / geometric series) in tests/test_oracle.py.

Extension beyond the reference: T == 1 is accepted (the reference fails on a
zero-length view, ref.py:23).
"""

from typing import Callable

import torch
import torch.nn.functional as F


def split(x: torch.Tensor):
    """Even-index and odd-index elements of a tree level (ref.py:8-24).

    >>> split(torch.tensor([1, 2, 3, 4, 5, 6, 7, 8])[None, None, :])
    (tensor([[[1, 3, 5, 7]]]), tensor([[[2, 4, 6, 8]]]))
    """
    return x[:, :, 0::2], x[:, :, 1::2]


def merge(lefts: torch.Tensor, rights: torch.Tensor) -> torch.Tensor:
    """Interleave two half-length levels into one (ref.py:27-46).

    >>> merge(torch.tensor([1, 3, 5, 7])[None, None, :], torch.tensor([2, 4, 6, 8])[None, None, :])
    tensor([[[1, 2, 3, 4, 5, 6, 7, 8]]])
    """
    return torch.stack((lefts, rights), dim=-1).flatten(-2)


def scan(
    gates: torch.Tensor,
    tokens: torch.Tensor,
    mul: Callable = torch.mul,
    add: Callable = torch.add,
    zeros_like: Callable = torch.zeros_like,
    ones_like: Callable = torch.ones_like,
    reverse: bool = False,
) -> torch.Tensor:
    """``x[t] = gates[t] * x[t-1] + tokens[t]`` (``x[t+1]`` when ``reverse``), shape (B, C, T).

    Signature and defaults as ref.py:49-57.
    """
    B, C, T = tokens.size()
    padded_T = 1 << max(T - 1, 0).bit_length()
    if padded_T != T:
        # identity elements (gate 1, token 0) at the END of the row (ref.py:78-82)
        gates = F.pad(gates, (0, padded_T - T), value=1).contiguous()
        tokens = F.pad(tokens, (0, padded_T - T), value=0).contiguous()

    levels = padded_T.bit_length() - 1  # int(log2(padded_T)), ref.py:84

    # Up-sweep (ref.py:100-109).  "near" is the child met first in scan order:
    # the even element going forward, the odd element going in reverse.
    g, x = gates, tokens
    near_children = []
    for _ in range(levels):
        g_even, g_odd = split(g)
        x_even, x_odd = split(x)
        if reverse:
            near_g, far_g, near_x, far_x = g_odd, g_even, x_odd, x_even
        else:
            near_g, far_g, near_x, far_x = g_even, g_odd, x_even, x_odd
        near_children.append((near_g, near_x))
        g = mul(near_g, far_g)
        x = add(mul(far_g, near_x), far_x)

    if levels == 0:
        state = zeros_like(tokens)
    else:
        # Root of the tree (ref.py:111-112), then the down-sweep (ref.py:116-121):
        # the near child inherits the parent's prefix, the far child gets prefix o near.
        prefix_g, prefix_x = ones_like(x), zeros_like(x)
        for near_g, near_x in reversed(near_children):
            far_prefix_g = mul(prefix_g, near_g)
            far_prefix_x = add(mul(prefix_x, near_g), near_x)
            if reverse:
                prefix_g = merge(far_prefix_g, prefix_g)
                prefix_x = merge(far_prefix_x, prefix_x)
            else:
                prefix_g = merge(prefix_g, far_prefix_g)
                prefix_x = merge(prefix_x, far_prefix_x)
        state = prefix_x  # exclusive scan: the state entering each step

    out = add(mul(state, gates), tokens)  # ref.py:86
    return out[:, :, :T]
