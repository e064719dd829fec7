"""``accelerated_scan.ref``: the reference's third import name (accelerated_scan/ref.py:49-57,
README.md:25-27 of the reference) served by the HIP kernels.

CPU tests: the module imports without a GPU, ``split`` / ``merge`` reproduce the
literals of ref.py:19-20,39-42, and ``scan`` refuses host tensors and custom
arithmetic instead of falling back to anything.  GPU tests: values and gradients,
forward and reverse, against the tree scan of oracle/ref_scan.py (the restatement
of the function this module stands in for) at the reference's tolerances
(tests/test_eq.py:13-14, tests/tests_eq_complex.py:23), and the reverse-scan
identity of tests/test_eq.py:65-90 run through this module on the device.
"""

import pytest
import torch

from oracle import ref_scan

DEVICE = "cuda"


def test_split_and_merge_literals():
    from accelerated_scan import ref

    x = torch.tensor([1, 2, 3, 4, 5, 6, 7, 8])[None, None, :]
    lefts, rights = ref.split(x)
    assert lefts.tolist() == [[[1, 3, 5, 7]]] and rights.tolist() == [[[2, 4, 6, 8]]]
    assert ref.merge(lefts, rights).tolist() == x.tolist()
    y = torch.randn(2, 3, 10)
    assert torch.equal(ref.merge(*ref.split(y)), y)
    for ours, theirs in zip(ref.split(y), ref_scan.split(y)):
        assert torch.equal(ours, theirs)


def test_no_cpu_path_and_no_custom_arithmetic():
    from accelerated_scan import ref

    gates, tokens = torch.rand(1, 2, 8), torch.rand(1, 2, 8)
    with pytest.raises(RuntimeError, match="device tensors"):
        ref.scan(gates, tokens)
    with pytest.raises(RuntimeError, match="device tensors"):
        ref.scan(gates, tokens, reverse=True)
    with pytest.raises(NotImplementedError):
        ref.scan(gates, tokens, mul=lambda a, b: a * b)


def _inputs(seed, B, C, T, dtype):
    gen = torch.Generator().manual_seed(seed)
    if dtype == torch.complex64:  # radius 0.4..1 as tests/tests_eq_complex.py:33-35 draws it
        gates = torch.polar(0.4 + 0.6 * torch.rand(B, C, T, generator=gen), 6.2831853 * torch.rand(B, C, T, generator=gen))
        tokens = torch.complex(torch.randn(B, C, T, generator=gen).tanh(), torch.randn(B, C, T, generator=gen).tanh())
    else:  # U(0,1) as tests/test_eq.py:16-19
        gates = torch.rand(B, C, T, generator=gen).to(dtype)
        tokens = torch.rand(B, C, T, generator=gen).to(dtype)
    return gates, tokens


TOL = {  # tests/test_eq.py:13-14, tests/tests_eq_complex.py:23
    torch.float32: dict(atol=1e-7, rtol=1.3e-6),
    torch.bfloat16: dict(atol=1e-1, rtol=1.6e-2),
    torch.float16: dict(atol=12e-3, rtol=1e-3),
    torch.complex64: dict(atol=1e-5, rtol=1e-4),
}


def _loss(out):
    # tests/test_eq.py:47 for the real dtypes; real and imaginary parts both weighted for complex64
    if out.is_complex():
        return (out.real + 0.5 * out.imag).mean(dim=-1).sum()
    return out.mean(dim=-1).sum()


@pytest.mark.gpu
@pytest.mark.parametrize("reverse", [False, True], ids=["forward", "reverse"])
@pytest.mark.parametrize("T", [32, 1000, 16323])
@pytest.mark.parametrize("dtype", list(TOL), ids=["fp32", "bf16", "fp16", "c64"])
def test_scan_matches_the_tree_scan(dtype, T, reverse):
    from accelerated_scan import ref

    gates, tokens = _inputs(3407 + T, 1, 96, T, dtype)
    g = gates.to(DEVICE).requires_grad_()
    x = tokens.to(DEVICE).requires_grad_()
    out = ref.scan(g, x, reverse=reverse)
    assert out.dtype == dtype and out.shape == x.shape
    _loss(out).backward()

    # the tree scan on the device in the same dtype, as the reference's tests run it (tests/test_eq.py:33,52)
    g_ref = gates.to(DEVICE).requires_grad_()
    x_ref = tokens.to(DEVICE).requires_grad_()
    out_ref = ref_scan.scan(g_ref, x_ref, reverse=reverse)
    _loss(out_ref).backward()

    tol = TOL[dtype]
    torch.testing.assert_close(out, out_ref, **tol)
    torch.testing.assert_close(x.grad, x_ref.grad, **tol)
    torch.testing.assert_close(g.grad, g_ref.grad, **tol)


@pytest.mark.gpu
@pytest.mark.parametrize("T", [2, 3, 64, 8000, 33753])
def test_reverse_scan_identity_of_the_reference(T):
    """tests/test_eq.py:65-90 through this module: the gradient of the token scan is the
    reverse scan of the incoming gradient over the gates shifted by one."""
    from accelerated_scan import ref

    gen = torch.Generator().manual_seed(1)
    f = torch.randn(1, 1, T, generator=gen).to(DEVICE).requires_grad_()
    x = torch.randn(1, 1, T, generator=gen).to(DEVICE).requires_grad_()
    c = ref.scan(f, x)
    dldc = torch.ones_like(c)
    fpx = torch.cat([f, torch.ones_like(f[:, :, :1])], dim=-1)[:, :, 1:].contiguous()
    dcdx = ref.scan(fpx.detach(), dldc, reverse=True)
    cp = torch.cat([torch.zeros_like(c[:, :, :1]), c], dim=-1)[:, :, :-1].contiguous()
    dcdf = dcdx * cp
    c.sum().backward()
    # randn gates grow products without bound as T grows: compare relative to the largest magnitude
    for got, want in ((x.grad, dcdx), (f.grad, dcdf.detach())):
        finite = torch.isfinite(want) & torch.isfinite(got)
        assert torch.equal(torch.isfinite(want), torch.isfinite(got))
        scale = want[finite].abs().max().item() if finite.any() else 1.0
        torch.testing.assert_close(got[finite], want[finite], atol=2e-5 * max(scale, 1.0), rtol=1.3e-6)
