"""torch.compile support: the operators are traced as opaque custom ops with
shape rules, forward and backward, and give the eager results."""

import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEVICE = "cuda"


def _inputs(T=3000, dtype=torch.float32):
    gen = torch.Generator().manual_seed(77)
    gates = torch.rand(2, 24, T, generator=gen).to(dtype).to(DEVICE).requires_grad_(True)
    tokens = torch.randn(2, 24, T, generator=gen).to(dtype).to(DEVICE).requires_grad_(True)
    weight = torch.randn(2, 24, T, generator=gen).to(dtype).to(DEVICE)
    return gates, tokens, weight


def test_opcheck_forward_and_backward_ops():
    from accelerated_scan import _ops

    gates, tokens, weight = _inputs(T=520)
    g, x = gates.detach(), tokens.detach()
    torch.library.opcheck(_ops.scan_forward, (g, x, False))
    torch.library.opcheck(_ops.scan_forward, (g, x, True))
    states = _ops.scan_forward(g, x, False)
    torch.library.opcheck(_ops.scan_backward, (g, states, weight, False))
    # complex gates with real tokens: complex states, real token gradient
    gc = torch.polar(g, x)
    sc = _ops.scan_forward(gc, x, False)
    assert sc.dtype == torch.complex64
    torch.library.opcheck(_ops.scan_forward, (gc, x, False))
    torch.library.opcheck(_ops.scan_backward, (gc, sc, torch.randn_like(sc), True))
    assert _ops.scan_backward(gc, sc, torch.randn_like(sc), True)[1].dtype == torch.float32


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
@pytest.mark.parametrize("module", ["warp", "scalar"])
def test_compiled_scan_matches_eager(module, backend):
    import importlib

    scan = importlib.import_module(f"accelerated_scan.{module}").scan

    def loss_fn(g, x, w):
        return (scan(g.sigmoid(), x) * w).sum()

    gates, tokens, weight = _inputs()
    loss_fn(gates, tokens, weight).backward()
    eager = (gates.grad.clone(), tokens.grad.clone())
    gates.grad = tokens.grad = None

    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    compiled(gates, tokens, weight).backward()
    # inductor fuses the sigmoid / multiply / sum around the opaque scan ops
    torch.testing.assert_close(gates.grad, eager[0], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(tokens.grad, eager[1], rtol=1e-5, atol=1e-5)


def test_compiled_complex_scan_matches_eager():
    from accelerated_scan.complex import scan

    gen = torch.Generator().manual_seed(5)
    shape = (1, 16, 2500)
    forget = torch.polar(0.9 + 0.1 * torch.rand(*shape, generator=gen),
                         2 * math.pi * torch.rand(*shape, generator=gen)).to(DEVICE).requires_grad_(True)
    inputs = torch.randn(*shape, generator=gen).to(DEVICE).requires_grad_(True)

    def loss_fn(f, i):
        return scan(f, i).abs().square().mean()

    loss_fn(forget, inputs).backward()
    eager = (forget.grad.clone(), inputs.grad.clone())
    forget.grad = inputs.grad = None
    compiled = torch.compile(loss_fn, backend="aot_eager", fullgraph=True)
    compiled(forget, inputs).backward()
    torch.testing.assert_close(forget.grad, eager[0], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(inputs.grad, eager[1], rtol=1e-5, atol=1e-6)


def test_opcheck_stateful_ops():
    from accelerated_scan import _ops

    gates, tokens, weight = _inputs(T=520)
    g, x = gates.detach(), tokens.detach()
    initial = torch.randn(2, 24, device=DEVICE)
    torch.library.opcheck(_ops.scan_forward_from, (g, x, initial, False))
    torch.library.opcheck(_ops.scan_forward_from, (g, x, initial, True))
    states = _ops.scan_forward_from(g, x, initial, False)
    torch.library.opcheck(_ops.scan_backward_from, (g, states, initial, weight, False))
    gc = torch.polar(g, x)
    ic = torch.complex(initial, initial.flip(0))
    sc = _ops.scan_forward_from(gc, x, ic, False)
    torch.library.opcheck(_ops.scan_backward_from, (gc, sc, ic, torch.randn_like(sc), True))
    d_gates, d_tokens, d_initial = _ops.scan_backward_from(gc, sc, ic, torch.randn_like(sc), True)
    assert d_tokens.dtype == torch.float32 and d_initial.dtype == torch.complex64 and d_initial.shape == ic.shape


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_chunked_scan_matches_eager(backend):
    """Two chunks with the state carried across, compiled as one graph."""
    from accelerated_scan.warp import scan

    def loss_fn(g, x, w, h0):
        g = g.sigmoid()
        half = g.shape[-1] // 2
        first = scan(g[..., :half].contiguous(), x[..., :half].contiguous(), h0)
        second = scan(g[..., half:].contiguous(), x[..., half:].contiguous(), first[..., -1])
        return (torch.cat([first, second], dim=-1) * w).sum()

    gates, tokens, weight = _inputs()
    h0 = torch.randn(2, 24, device=DEVICE, requires_grad=True)
    loss_fn(gates, tokens, weight, h0).backward()
    eager = (gates.grad.clone(), tokens.grad.clone(), h0.grad.clone())
    gates.grad = tokens.grad = h0.grad = None

    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    compiled(gates, tokens, weight, h0).backward()
    torch.testing.assert_close(gates.grad, eager[0], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(tokens.grad, eager[1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h0.grad, eager[2], rtol=1e-5, atol=1e-5)
