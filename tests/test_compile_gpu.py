"""torch.compile support: the operators are traced as opaque custom ops with
shape rules, forward and backward.  Compiled and eager results are both checked
against the oracle (the tree scan of oracle/ref_scan.py differentiated by
autograd, or the fp64 loops of oracle/seqscan.c), and against each other."""

import math

import numpy as np
import pytest
import torch

from oracle import ref_scan, seqscan

pytestmark = pytest.mark.gpu

DEVICE = "cuda"


def _oracle_grads(loss_fn, *tensors):
    """Gradients of ``loss_fn`` (written over the tree scan) for fresh copies of the leaves."""
    leaves = [t.detach().clone().requires_grad_(t.requires_grad) for t in tensors]
    loss_fn(*leaves).backward()
    return [leaf.grad for leaf in leaves if leaf.requires_grad]


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
    # leaves that require gradients: also checks the autograd registration and the traced backward
    torch.library.opcheck(_ops.scan_forward, (gates, tokens, False))
    torch.library.opcheck(_ops.scan_forward, (gates, tokens, True))
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

    def loss_fn(g, x, w, scan=scan):
        return (scan(g.sigmoid(), x) * w).sum()

    gates, tokens, weight = _inputs()
    want = _oracle_grads(lambda g, x, w: loss_fn(g, x, w, scan=ref_scan.scan), gates, tokens, weight)
    out_want = ref_scan.scan(gates.detach().sigmoid(), tokens.detach())

    loss_fn(gates, tokens, weight).backward()
    eager = (gates.grad.clone(), tokens.grad.clone())
    gates.grad = tokens.grad = None
    torch.testing.assert_close(eager[0], want[0], rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(eager[1], want[1], rtol=1e-4, atol=1e-4)

    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    compiled(gates, tokens, weight).backward()
    # inductor fuses the sigmoid / multiply / sum around the opaque scan ops
    torch.testing.assert_close(gates.grad, eager[0], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(tokens.grad, eager[1], rtol=1e-5, atol=1e-5)
    # against the oracle: the tree scan, differentiated by autograd (sums of 3000 terms in another order)
    torch.testing.assert_close(gates.grad, want[0], rtol=1e-4, atol=1e-4)
    torch.testing.assert_close(tokens.grad, want[1], rtol=1e-4, atol=1e-4)
    out = torch.compile(lambda g, x: scan(g.sigmoid(), x), backend=backend, fullgraph=True)(
        gates.detach(), tokens.detach())
    torch.testing.assert_close(out, out_want, rtol=1e-5, atol=1e-5)


def test_compiled_complex_scan_matches_eager():
    from accelerated_scan.complex import scan

    gen = torch.Generator().manual_seed(5)
    shape = (1, 16, 2500)
    forget = torch.polar(0.9 + 0.1 * torch.rand(*shape, generator=gen),
                         2 * math.pi * torch.rand(*shape, generator=gen)).to(DEVICE).requires_grad_(True)
    inputs = torch.randn(*shape, generator=gen).to(DEVICE).requires_grad_(True)

    def loss_fn(f, i, scan=scan):
        return scan(f, i).abs().square().mean()

    # oracle: the tree scan over the inputs promoted to complex, as complex.py:162,168-169 does
    want = _oracle_grads(lambda f, i: loss_fn(f, i, scan=lambda a, b: ref_scan.scan(a, b.to(a.dtype))),
                         forget, inputs)
    loss_fn(forget, inputs).backward()
    eager = (forget.grad.clone(), inputs.grad.clone())
    forget.grad = inputs.grad = None
    compiled = torch.compile(loss_fn, backend="aot_eager", fullgraph=True)
    compiled(forget, inputs).backward()
    torch.testing.assert_close(forget.grad, eager[0], rtol=1e-5, atol=1e-6)
    torch.testing.assert_close(inputs.grad, eager[1], rtol=1e-5, atol=1e-6)
    for got in (eager, (forget.grad, inputs.grad)):
        torch.testing.assert_close(got[0], want[0], rtol=1e-4, atol=1e-5)  # tests/tests_eq_complex.py:23
        torch.testing.assert_close(got[1], want[1], rtol=1e-4, atol=1e-5)


def test_opcheck_stateful_ops():
    from accelerated_scan import _ops

    gates, tokens, weight = _inputs(T=520)
    g, x = gates.detach(), tokens.detach()
    initial = torch.randn(2, 24, device=DEVICE)
    torch.library.opcheck(_ops.scan_forward_from, (g, x, initial, False))
    torch.library.opcheck(_ops.scan_forward_from, (g, x, initial, True))
    states = _ops.scan_forward_from(g, x, initial, False)
    torch.library.opcheck(_ops.scan_backward_from, (g, states, initial, weight, False))
    reverse_states = _ops.scan_forward_from(g, x, initial, True)
    torch.library.opcheck(_ops.scan_backward_reverse, (g, reverse_states, initial, weight, False))
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

    def oracle_loss(g, x, w, h0):
        # a scan from h0 is the zero-start scan of tokens whose first element carries gate[0] * h0
        g = g.sigmoid()
        x = torch.cat([(x[..., 0] + g[..., 0] * h0)[..., None], x[..., 1:]], dim=-1)
        return (ref_scan.scan(g, x) * w).sum()

    gates, tokens, weight = _inputs()
    h0 = torch.randn(2, 24, device=DEVICE, requires_grad=True)
    want = _oracle_grads(oracle_loss, gates, tokens, weight, h0)
    loss_fn(gates, tokens, weight, h0).backward()
    eager = (gates.grad.clone(), tokens.grad.clone(), h0.grad.clone())
    gates.grad = tokens.grad = h0.grad = None
    for got, ref in zip(eager, want):
        torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-4)

    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    compiled(gates, tokens, weight, h0).backward()
    torch.testing.assert_close(gates.grad, eager[0], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(tokens.grad, eager[1], rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(h0.grad, eager[2], rtol=1e-5, atol=1e-5)
    for got, ref in zip((gates.grad, tokens.grad, h0.grad), want):
        torch.testing.assert_close(got, ref, rtol=1e-4, atol=1e-4)


# ---------------------------------------------------------------------------
# The forward operators are differentiable on their own (register_autograd):
# no autograd.Function around them, eager and compiled, against the fp64 loops.
# ---------------------------------------------------------------------------
def _np(t):
    return t.detach().cpu().numpy()


def _assert_np(got, want, what, tol=2e-5):
    want = np.asarray(want)
    scale = max(1.0, float(np.abs(want).max()))
    np.testing.assert_allclose(_np(got), want, rtol=tol, atol=tol * scale, err_msg=what)


@pytest.mark.parametrize("mode", ["eager", "aot_eager", "inductor"])
@pytest.mark.parametrize("reverse", [False, True], ids=["forward", "reverse"])
def test_scan_forward_op_is_differentiable(mode, reverse):
    op = torch.ops.accelerated_scan.scan_forward
    gates, tokens, weight = _inputs(T=2100)

    def run(g, x, w):
        out = op(g, x, reverse)
        return out, (out * w).sum()

    if mode != "eager":
        run = torch.compile(run, backend=mode, fullgraph=True)
    out, loss = run(gates, tokens, weight)
    dg, dx = torch.autograd.grad(loss, (gates, tokens))
    g2, x2, w2 = (_np(t).reshape(48, -1) for t in (gates, tokens, weight))
    t_out = seqscan.forward(g2, x2, reverse=reverse)
    _assert_np(out.reshape(48, -1), t_out, "states")
    if reverse:  # the reverse scan is the forward scan of the flipped rows
        t_dg, t_dx = seqscan.backward(g2[:, ::-1].copy(), _np(out).reshape(48, -1)[:, ::-1].copy(), w2[:, ::-1].copy())
        t_dg, t_dx = t_dg[:, ::-1], t_dx[:, ::-1]
    else:
        t_dg, t_dx = seqscan.backward(g2, _np(out).reshape(48, -1), w2)
    _assert_np(dg.reshape(48, -1), t_dg, "d_gates")
    _assert_np(dx.reshape(48, -1), t_dx, "d_tokens")


@pytest.mark.parametrize("mode", ["eager", "aot_eager"])  # inductor generates no code for complex elementwise ops
def test_scan_forward_op_complex_gates_real_tokens_gradients(mode):
    op = torch.ops.accelerated_scan.scan_forward
    gen = torch.Generator().manual_seed(9)
    rows, T = 12, 1500
    gates = torch.polar(0.6 + 0.4 * torch.rand(1, rows, T, generator=gen),
                        2 * math.pi * torch.rand(1, rows, T, generator=gen)).to(DEVICE).requires_grad_(True)
    tokens = torch.randn(1, rows, T, generator=gen).to(DEVICE).requires_grad_(True)
    weight = torch.complex(torch.randn(1, rows, T, generator=gen), torch.randn(1, rows, T, generator=gen)).to(DEVICE)

    def run(g, x, w):
        out = op(g, x, False)
        # real loss whose gradient with respect to out is w (torch's convention for complex leaves)
        return out, (out * w.conj()).real.sum()

    if mode != "eager":
        run = torch.compile(run, backend=mode, fullgraph=True)
    out, loss = run(gates, tokens, weight)
    dg, dx = torch.autograd.grad(loss, (gates, tokens))
    assert dx.dtype == torch.float32 and dg.dtype == torch.complex64
    g2 = _np(gates).reshape(rows, T)
    t_out = seqscan.forward(g2, _np(tokens).reshape(rows, T).astype(np.complex64))
    _assert_np(out.reshape(rows, T), t_out, "states")
    t_dg, t_dx = seqscan.backward(g2, _np(out).reshape(rows, T), _np(weight).reshape(rows, T))
    _assert_np(dg.reshape(rows, T), t_dg, "d_gates")
    _assert_np(dx.reshape(rows, T), t_dx.real, "d_tokens")


@pytest.mark.parametrize("mode", ["eager", "inductor"])
@pytest.mark.parametrize("reverse", [False, True], ids=["forward", "reverse"])
def test_scan_forward_from_op_is_differentiable(mode, reverse):
    op = torch.ops.accelerated_scan.scan_forward_from
    gates, tokens, weight = _inputs(T=1700)
    initial = torch.randn(2, 24, device=DEVICE, requires_grad=True)

    def run(g, x, h, w):
        out = op(g, x, h, reverse)
        return out, (out * w).sum()

    if mode != "eager":
        run = torch.compile(run, backend=mode, fullgraph=True)
    out, loss = run(gates, tokens, initial, weight)
    dg, dx, dh = torch.autograd.grad(loss, (gates, tokens, initial))
    g2, x2, w2 = (_np(t).reshape(48, -1) for t in (gates, tokens, weight))
    h2 = _np(initial).reshape(48)
    _assert_np(out.reshape(48, -1), seqscan.forward_from(g2, x2, h2, reverse=reverse), "states")
    o2 = _np(out).reshape(48, -1)
    if reverse:
        t_dg, t_dx, t_dh = seqscan.backward_from(g2[:, ::-1].copy(), o2[:, ::-1].copy(), h2, w2[:, ::-1].copy())
        t_dg, t_dx = t_dg[:, ::-1], t_dx[:, ::-1]
    else:
        t_dg, t_dx, t_dh = seqscan.backward_from(g2, o2, h2, w2)
    _assert_np(dg.reshape(48, -1), t_dg, "d_gates")
    _assert_np(dx.reshape(48, -1), t_dx, "d_tokens")
    _assert_np(dh.reshape(48), t_dh, "d_initial")


@pytest.mark.parametrize("mode", ["eager", "inductor"])
def test_scan_forward_gated_op_is_differentiable(mode):
    from accelerated_scan import _abi

    op = torch.ops.accelerated_scan.scan_forward_gated
    gates, tokens, weight = _inputs(T=1300)
    logits = (4 * gates.detach() - 1).requires_grad_(True)
    initial = torch.randn(2, 24, device=DEVICE, requires_grad=True)

    def run(z, x, h, w):
        out = op(z, x, h, _abi.GATE_SIGMOID)
        return out, (out * w).sum()

    if mode != "eager":
        run = torch.compile(run, backend=mode, fullgraph=True)
    out, loss = run(logits, tokens, initial, weight)
    dz, dx, dh = torch.autograd.grad(loss, (logits, tokens, initial))
    z2, x2, w2 = (_np(t).reshape(48, -1) for t in (logits, tokens, weight))
    h2 = _np(initial).reshape(48)
    _assert_np(out.reshape(48, -1), seqscan.forward_sigmoid(z2, x2, h2), "states")
    t_dz, t_dx, t_dh = seqscan.backward_sigmoid(z2, _np(out).reshape(48, -1), w2, h2)
    _assert_np(dz.reshape(48, -1), t_dz, "d_gate_logits")
    _assert_np(dx.reshape(48, -1), t_dx, "d_tokens")
    _assert_np(dh.reshape(48), t_dh, "d_initial")


def test_ops_validate_their_arguments():
    """The operators are public as torch.ops.accelerated_scan.*: a shape mismatch
    must be an error, not a write past the end of the output."""
    from accelerated_scan import _ops

    g = torch.rand(2, 3, 64, device=DEVICE)
    with pytest.raises(RuntimeError, match="one shape"):
        _ops.scan_forward(g, torch.rand(2, 3, 128, device=DEVICE), False)
    with pytest.raises(RuntimeError, match="contiguous"):
        _ops.scan_forward(g, torch.rand(2, 3, 128, device=DEVICE)[..., ::2], False)
    with pytest.raises(RuntimeError, match="device tensors"):
        _ops.scan_forward(g.cpu(), g.cpu(), False)
    with pytest.raises(RuntimeError, match="dtype"):
        _ops.scan_backward(g, g.half(), g, False)
    with pytest.raises(RuntimeError, match="state of shape"):
        _ops.scan_forward_from(g, g, torch.rand(2, 4, device=DEVICE), False)
    with pytest.raises(RuntimeError, match="expecting one dtype"):
        _ops.scan_forward(g, g.half(), False)
