"""CPU tests that pin the oracle (oracle/ref_scan.py, oracle/seqscan.c).

Three independent anchors:
  * golden outputs recorded from the reference's own tree scan (bit-exact for
    the forward values, tight tolerance for autograd gradients);
  * the sequential recurrence in fp64 (different algorithm, different language);
  * closed forms that reduce the operator to library routines (cumsum, cumprod,
    geometric series) and the flip identity for the reverse scan.
The backward formulas are pinned the way the reference proves them
(tests/test_eq.py:65-90) and by autograd through an explicit fp64 loop.
"""

import doctest
import math

import numpy as np
import pytest
import torch

from oracle import ref_scan, seqscan

SEQLENS = [2**i for i in range(5, 13)] + [8000, 16323]

REAL_CASES = ["cfg1_fwd", "pow2_rev", "pad_fwd", "pad_rev", "tiny_T2", "tiny_T3", "long_memory",
              "grads_fwd", "grads_pow2"]


def test_doctests():
    assert doctest.testmod(ref_scan).failed == 0


@pytest.mark.parametrize("name", REAL_CASES)
def test_tree_scan_bit_exact_vs_reference_golden(golden, name):
    gates = torch.from_numpy(golden[f"{name}.gates"])
    tokens = torch.from_numpy(golden[f"{name}.tokens"])
    reverse = bool(golden[f"{name}.reverse"])
    out = ref_scan.scan(gates, tokens, reverse=reverse)
    assert torch.equal(out, torch.from_numpy(golden[f"{name}.out"]))


@pytest.mark.parametrize("name", ["grads_fwd", "grads_pow2"])
def test_tree_scan_gradients_vs_reference_golden(golden, name):
    gates = torch.from_numpy(golden[f"{name}.gates"]).requires_grad_(True)
    tokens = torch.from_numpy(golden[f"{name}.tokens"]).requires_grad_(True)
    grad_out = torch.from_numpy(golden[f"{name}.grad_out"])
    out = ref_scan.scan(gates, tokens)
    dg, dt = torch.autograd.grad(out, (gates, tokens), grad_out)
    # same graph up to the order in which autograd sums a node's contributions
    torch.testing.assert_close(dg, torch.from_numpy(golden[f"{name}.d_gates"]), atol=1e-6, rtol=1e-6)
    torch.testing.assert_close(dt, torch.from_numpy(golden[f"{name}.d_tokens"]), atol=1e-6, rtol=1e-6)


@pytest.mark.parametrize("name", ["complex_real_tokens", "complex_complex_tokens"])
def test_tree_scan_complex_vs_reference_golden(golden, name):
    gates = torch.from_numpy(golden[f"{name}.gates"]).requires_grad_(True)
    tokens = torch.from_numpy(golden[f"{name}.tokens"]).requires_grad_(True)
    grad_out = torch.from_numpy(golden[f"{name}.grad_out"])
    out = ref_scan.scan(gates, tokens)
    assert torch.equal(out.detach(), torch.from_numpy(golden[f"{name}.out"]))
    dg, dt = torch.autograd.grad(out, (gates, tokens), grad_out)
    torch.testing.assert_close(dg, torch.from_numpy(golden[f"{name}.d_gates"]), atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(dt, torch.from_numpy(golden[f"{name}.d_tokens"]), atol=1e-5, rtol=1e-5)


@pytest.mark.parametrize("name", REAL_CASES + ["complex_real_tokens", "complex_complex_tokens"])
def test_sequential_fp64_vs_reference_golden(golden, name):
    """The C loops agree with the reference's recorded outputs to fp32 rounding."""
    gates = golden[f"{name}.gates"]
    tokens = golden[f"{name}.tokens"]
    reverse = bool(golden.get(f"{name}.reverse", 0))
    truth = seqscan.forward(gates, tokens, reverse=reverse)
    ref = golden[f"{name}.out"]
    scale = np.abs(truth).max()
    assert np.abs(truth - ref).max() <= 2e-6 * scale
    if f"{name}.d_gates" in golden:
        if np.iscomplexobj(gates) and not np.iscomplexobj(tokens):
            tokens_c = tokens.astype(np.complex64)
        states = seqscan.forward(gates, tokens).astype(gates.dtype)
        dg, dt = seqscan.backward(gates, states, golden[f"{name}.grad_out"])
        ref_dt = golden[f"{name}.d_tokens"]
        if not np.iscomplexobj(ref_dt) and np.iscomplexobj(dt):
            dt = dt.real  # real tokens keep the real part (accelerated_scan/complex.py:217-218)
        assert np.abs(dt - ref_dt).max() <= 1e-5 * np.abs(dt).max()
        assert np.abs(dg - golden[f"{name}.d_gates"]).max() <= 1e-5 * np.abs(dg).max()


@pytest.mark.parametrize("T", [1, 2, 3, 5, 31, 32, 33, 100, 1024, 1025, 4097])
@pytest.mark.parametrize("reverse", [False, True])
def test_tree_scan_vs_sequential_fp64(T, reverse):
    gen = torch.Generator().manual_seed(T)
    gates = torch.rand(2, 3, T, generator=gen)
    tokens = torch.randn(2, 3, T, generator=gen)
    out = ref_scan.scan(gates, tokens, reverse=reverse).numpy()
    truth = seqscan.forward(gates.numpy(), tokens.numpy(), reverse=reverse)
    np.testing.assert_allclose(out, truth, rtol=2e-6, atol=2e-6)


def test_closed_forms():
    gen = torch.Generator().manual_seed(0)
    T = 777
    tokens = torch.randn(1, 4, T, generator=gen, dtype=torch.float64)
    gates = 0.5 + torch.rand(1, 4, T, generator=gen, dtype=torch.float64)
    ones, zeros = torch.ones_like(tokens), torch.zeros_like(tokens)
    # gates == 1: running sum
    torch.testing.assert_close(ref_scan.scan(ones, tokens), torch.cumsum(tokens, -1), rtol=1e-12, atol=1e-12)
    # gates == 0: the tokens themselves
    assert torch.equal(ref_scan.scan(zeros, tokens), tokens)
    # tokens == 0: zero
    assert torch.equal(ref_scan.scan(gates, zeros), zeros)
    # impulse at t = 0: running product of gates[1:]
    impulse = zeros.clone()
    impulse[..., 0] = 1.0
    g1 = gates.clone()
    g1[..., 0] = 1.0
    torch.testing.assert_close(ref_scan.scan(gates, impulse), torch.cumprod(g1, -1), rtol=1e-12, atol=0)
    # constant gate a, tokens == 1: (1 - a^(t+1)) / (1 - a)
    a = 0.9
    t = torch.arange(T, dtype=torch.float64)
    closed = (1 - a ** (t + 1)) / (1 - a)
    got = ref_scan.scan(torch.full_like(tokens, a), ones)
    torch.testing.assert_close(got, closed.expand_as(got), rtol=1e-12, atol=0)
    # and the same through the C loop (fp32 inputs)
    seq = seqscan.forward(np.full((1, T), 0.5, np.float32), np.ones((1, T), np.float32))
    np.testing.assert_allclose(seq[0], (1 - 0.5 ** (np.arange(T) + 1.0)) / 0.5, rtol=1e-15)
    seq = seqscan.forward(np.ones((2, T), np.float32), tokens[0, :2].float().numpy())
    np.testing.assert_allclose(seq, np.cumsum(tokens[0, :2].float().numpy().astype(np.float64), -1), rtol=1e-12)


@pytest.mark.parametrize("T", [2, 7, 64, 1000])
def test_reverse_is_flip_of_forward(T):
    gen = torch.Generator().manual_seed(T)
    gates = torch.rand(1, 3, T, generator=gen, dtype=torch.float64)
    tokens = torch.randn(1, 3, T, generator=gen, dtype=torch.float64)
    rev = ref_scan.scan(gates, tokens, reverse=True)
    fwd = ref_scan.scan(gates.flip(-1).contiguous(), tokens.flip(-1).contiguous()).flip(-1)
    torch.testing.assert_close(rev, fwd, rtol=1e-12, atol=1e-12)
    truth = seqscan.forward(gates.float().numpy(), tokens.float().numpy(), reverse=True)
    truth_flip = seqscan.forward(gates.float().numpy()[..., ::-1], tokens.float().numpy()[..., ::-1])[..., ::-1]
    np.testing.assert_array_equal(truth, truth_flip)


@pytest.mark.parametrize("seqlen", SEQLENS)
def test_backward_is_shifted_reverse_scan(seqlen):
    """The identity the reference proves at tests/test_eq.py:65-90, same tolerances."""
    gen = torch.Generator().manual_seed(1)
    f = torch.randn(1, 1, seqlen, generator=gen, requires_grad=True)
    x = torch.randn(1, 1, seqlen, generator=gen, requires_grad=True)
    c = ref_scan.scan(f, x)
    ones = torch.ones_like(c)
    f_shift = torch.cat([f, torch.ones_like(f[:, :, :1])], dim=-1)[:, :, 1:].contiguous()
    dcdx = ref_scan.scan(f_shift, ones, reverse=True)
    c_shift = torch.cat([torch.zeros_like(c[:, :, :1]), c], dim=-1)[:, :, :-1].contiguous()
    dcdf = dcdx * c_shift
    c.sum().backward()
    torch.testing.assert_close(x.grad, dcdx, atol=1e-5, rtol=1.3e-6)
    torch.testing.assert_close(f.grad, dcdf, atol=2e-5, rtol=1.3e-6)


def _loop_scan(gates, tokens):
    """The recurrence as an explicit Python loop (autograd-friendly, any dtype)."""
    state = torch.zeros_like(tokens[..., 0])
    outs = []
    for t in range(tokens.shape[-1]):
        state = gates[..., t] * state + tokens[..., t]
        outs.append(state)
    return torch.stack(outs, dim=-1)


@pytest.mark.parametrize("T", [1, 2, 9, 130])
def test_sequential_backward_vs_autograd_of_loop(T):
    gen = torch.Generator().manual_seed(100 + T)
    gates = torch.rand(2, 2, T, generator=gen)
    tokens = torch.randn(2, 2, T, generator=gen)
    grad_out = torch.randn(2, 2, T, generator=gen)
    g64 = gates.double().requires_grad_(True)
    t64 = tokens.double().requires_grad_(True)
    out = _loop_scan(g64, t64)
    dg_ref, dt_ref = torch.autograd.grad(out, (g64, t64), grad_out.double())
    states = seqscan.forward(gates.numpy(), tokens.numpy()).astype(np.float32)
    dg, dt = seqscan.backward(gates.numpy(), states, grad_out.numpy())
    np.testing.assert_allclose(dt, dt_ref.numpy(), rtol=1e-12, atol=1e-12)
    # states were rounded to fp32 before the multiply
    np.testing.assert_allclose(dg, dg_ref.numpy(), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("T", [1, 2, 9, 130])
@pytest.mark.parametrize("real_tokens", [False, True])
def test_sequential_complex_backward_vs_autograd_of_loop(T, real_tokens):
    gen = torch.Generator().manual_seed(200 + T)
    angle = 2 * math.pi * torch.rand(1, 3, T, generator=gen)
    radius = 0.9 + 0.1 * torch.rand(1, 3, T, generator=gen)
    gates = torch.polar(radius, angle)
    if real_tokens:
        tokens = torch.randn(1, 3, T, generator=gen)
    else:
        tokens = torch.complex(torch.randn(1, 3, T, generator=gen), torch.randn(1, 3, T, generator=gen))
    grad_out = torch.complex(torch.randn(1, 3, T, generator=gen), torch.randn(1, 3, T, generator=gen))
    g128 = gates.to(torch.complex128).requires_grad_(True)
    t128 = (tokens.double() if real_tokens else tokens.to(torch.complex128)).requires_grad_(True)
    out = _loop_scan(g128, t128.to(torch.complex128))
    dg_ref, dt_ref = torch.autograd.grad(out, (g128, t128), grad_out.to(torch.complex128))
    fwd = seqscan.forward(gates.numpy(), tokens.numpy().astype(np.complex64))
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    dg, dt = seqscan.backward(gates.numpy(), fwd.astype(np.complex64), grad_out.numpy())
    if real_tokens:
        dt = dt.real
    np.testing.assert_allclose(dt, dt_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dg, dg_ref.numpy(), rtol=1e-5, atol=1e-5)


def test_tree_scan_complex_vs_sequential():
    gen = torch.Generator().manual_seed(3)
    T = 1000
    gates = torch.polar(0.99 + 0.01 * torch.rand(1, 4, T, generator=gen), 2 * math.pi * torch.rand(1, 4, T, generator=gen))
    tokens = torch.randn(1, 4, T, generator=gen).tanh()
    out = ref_scan.scan(gates, tokens).numpy()
    truth = seqscan.forward(gates.numpy(), tokens.numpy().astype(np.complex64))
    np.testing.assert_allclose(out, truth, rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------------------
# Scans started from a given state (oracle functions *_from)
# ---------------------------------------------------------------------------
def _loop_scan_from(gates, tokens, initial, reverse=False):
    state = initial
    outs = [None] * gates.shape[-1]
    order = range(gates.shape[-1] - 1, -1, -1) if reverse else range(gates.shape[-1])
    for t in order:
        state = gates[..., t] * state + tokens[..., t]
        outs[t] = state
    return torch.stack(outs, dim=-1)


def _complex_inputs(gen, shape):
    gates = torch.polar(0.9 + 0.1 * torch.rand(*shape, generator=gen), 2 * math.pi * torch.rand(*shape, generator=gen))
    tokens = torch.complex(torch.randn(*shape, generator=gen), torch.randn(*shape, generator=gen))
    grad_out = torch.complex(torch.randn(*shape, generator=gen), torch.randn(*shape, generator=gen))
    initial = torch.complex(torch.randn(*shape[:-1], generator=gen), torch.randn(*shape[:-1], generator=gen))
    return gates, tokens, grad_out, initial


@pytest.mark.parametrize("cplx", [False, True])
def test_from_zero_equals_zero_start(cplx):
    gen = torch.Generator().manual_seed(7)
    if cplx:
        gates, tokens, grad_out, initial = (t.numpy() for t in _complex_inputs(gen, (2, 3, 77)))
    else:
        gates, tokens, grad_out = (torch.randn(2, 3, 77, generator=gen).numpy() for _ in range(3))
        initial = np.zeros((2, 3), dtype=np.float32)
    zero = np.zeros_like(initial)
    for reverse in (False, True):
        np.testing.assert_array_equal(seqscan.forward_from(gates, tokens, zero, reverse),
                                      seqscan.forward(gates, tokens, reverse))
    states = seqscan.forward(gates, tokens).astype(gates.dtype)
    dg, dx, di = seqscan.backward_from(gates, states, zero, grad_out)
    dg0, dx0 = seqscan.backward(gates, states, grad_out)
    np.testing.assert_array_equal(dg, dg0)
    np.testing.assert_array_equal(dx, dx0)
    np.testing.assert_allclose(di, np.conj(gates[..., 0].astype(di.dtype)) * dx0[..., 0], rtol=1e-14)


@pytest.mark.parametrize("cplx", [False, True])
@pytest.mark.parametrize("cut", [1, 50, 129])
def test_from_chunking_identity(cplx, cut):
    """A scan cut in two, the second part started from the last state of the
    first, is the uncut scan; gradients chain through d_initial."""
    gen = torch.Generator().manual_seed(11 + cut)
    T = 130
    if cplx:
        gates, tokens, grad_out, _ = (t.numpy() for t in _complex_inputs(gen, (2, 2, T)))
    else:
        gates = torch.rand(2, 2, T, generator=gen).numpy()
        tokens, grad_out = (torch.randn(2, 2, T, generator=gen).numpy() for _ in range(2))
    whole = seqscan.forward(gates, tokens)
    first = seqscan.forward(gates[..., :cut], tokens[..., :cut])
    carry = first[..., -1].astype(gates.dtype)  # handed over in storage precision
    second = seqscan.forward_from(gates[..., cut:], tokens[..., cut:], carry)
    np.testing.assert_allclose(second, whole[..., cut:], rtol=2e-6, atol=2e-6)

    # gradients, with exact (fp32-representable) states so the identity is tight
    states = whole.astype(gates.dtype)
    dg, dx = seqscan.backward(gates, states, grad_out)
    dg2, dx2, di2 = seqscan.backward_from(gates[..., cut:], states[..., cut:], states[..., cut - 1], grad_out[..., cut:])
    np.testing.assert_allclose(dg2, dg[..., cut:], rtol=1e-13, atol=1e-13)
    np.testing.assert_allclose(dx2, dx[..., cut:], rtol=1e-13, atol=1e-13)
    # the adjoint entering the first part at its last step is grad_out there plus d_initial of the second part
    np.testing.assert_allclose(grad_out[..., cut - 1] + di2, dx[..., cut - 1], rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("T", [1, 2, 9, 64])
@pytest.mark.parametrize("cplx", [False, True])
def test_from_vs_autograd_of_loop(T, cplx):
    gen = torch.Generator().manual_seed(300 + T)
    if cplx:
        gates, tokens, grad_out, initial = _complex_inputs(gen, (2, 2, T))
        wide = torch.complex128
    else:
        gates = torch.rand(2, 2, T, generator=gen)
        tokens, grad_out = (torch.randn(2, 2, T, generator=gen) for _ in range(2))
        initial = torch.randn(2, 2, generator=gen)
        wide = torch.float64
    gw, tw, iw = (t.to(wide).requires_grad_(True) for t in (gates, tokens, initial))
    out = _loop_scan_from(gw, tw, iw)
    dg_ref, dt_ref, di_ref = torch.autograd.grad(out, (gw, tw, iw), grad_out.to(wide))
    fwd = seqscan.forward_from(gates.numpy(), tokens.numpy(), initial.numpy())
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    rev = seqscan.forward_from(gates.numpy(), tokens.numpy(), initial.numpy(), reverse=True)
    np.testing.assert_allclose(rev, _loop_scan_from(gw, tw, iw, reverse=True).detach().numpy(), rtol=1e-12, atol=1e-12)
    dg, dt, di = seqscan.backward_from(gates.numpy(), fwd.astype(gates.numpy().dtype), initial.numpy(), grad_out.numpy())
    np.testing.assert_allclose(dt, dt_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(di, di_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dg, dg_ref.numpy(), rtol=1e-5, atol=1e-5)  # states rounded to fp32 before the multiply
    # the reverse scan's gradients against autograd through the loop run from the last element down
    out_rev = _loop_scan_from(gw, tw, iw, reverse=True)
    rdg_ref, rdt_ref, rdi_ref = torch.autograd.grad(out_rev, (gw, tw, iw), grad_out.to(wide))
    rdg, rdt, rdi = seqscan.backward_from(gates.numpy(), rev.astype(gates.numpy().dtype), initial.numpy(), grad_out.numpy(),
                                          reverse=True)
    np.testing.assert_allclose(rdt, rdt_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(rdi, rdi_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(rdg, rdg_ref.numpy(), rtol=1e-5, atol=1e-5)


# ---------------------------------------------------------------------------
# Sigmoid-gated scans (oracle functions *_sigmoid)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 2, 9, 64])
@pytest.mark.parametrize("with_initial", [False, True])
def test_sigmoid_vs_autograd_of_loop(T, with_initial):
    gen = torch.Generator().manual_seed(400 + T)
    logits = 3.0 * torch.randn(2, 2, T, generator=gen)
    tokens, grad_out = (torch.randn(2, 2, T, generator=gen) for _ in range(2))
    initial = torch.randn(2, 2, generator=gen) if with_initial else torch.zeros(2, 2)
    zw, tw, iw = (t.double().requires_grad_(True) for t in (logits, tokens, initial))
    out = _loop_scan_from(torch.sigmoid(zw), tw, iw)
    dz_ref, dt_ref, di_ref = torch.autograd.grad(out, (zw, tw, iw), grad_out.double())
    init_arg = initial.numpy() if with_initial else None
    fwd = seqscan.forward_sigmoid(logits.numpy(), tokens.numpy(), init_arg)
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    dz, dt, di = seqscan.backward_sigmoid(logits.numpy(), fwd.astype(np.float32), grad_out.numpy(), init_arg)
    np.testing.assert_allclose(dt, dt_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(di, di_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dz, dz_ref.numpy(), rtol=1e-5, atol=1e-5)  # states rounded to fp32 before the multiply


def test_sigmoid_vs_plain_scan_of_rounded_gates_and_closed_form():
    gen = torch.Generator().manual_seed(17)
    logits = 2.0 * torch.randn(3, 4, 200, generator=gen)
    tokens, grad_out = (torch.randn(3, 4, 200, generator=gen) for _ in range(2))
    gates = torch.sigmoid(logits.double())
    fwd = seqscan.forward_sigmoid(logits.numpy(), tokens.numpy())
    plain = seqscan.forward(gates.float().numpy(), tokens.numpy())
    np.testing.assert_allclose(fwd, plain, rtol=1e-5, atol=1e-5)  # gates rounded to fp32 on one side
    states = fwd.astype(np.float32)
    dz, dx, _ = seqscan.backward_sigmoid(logits.numpy(), states, grad_out.numpy())
    dg, dx_plain = seqscan.backward(gates.float().numpy(), states, grad_out.numpy())
    np.testing.assert_allclose(dx, dx_plain, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dz, dg * (gates * (1 - gates)).numpy(), rtol=1e-5, atol=1e-5)
    # z = 0: every gate is 1/2, unit tokens give 2 - 2^-t
    T = 30
    out = seqscan.forward_sigmoid(np.zeros((1, 1, T), np.float32), np.ones((1, 1, T), np.float32))
    np.testing.assert_allclose(out[0, 0], 2.0 - 0.5 ** np.arange(T), rtol=1e-15)
    # saturated gates: z = +40 is a running sum, z = -40 returns the tokens
    x = tokens[:1, :1, :50].numpy()
    np.testing.assert_allclose(seqscan.forward_sigmoid(np.full_like(x, 40.0), x), np.cumsum(x.astype(np.float64), -1), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(seqscan.forward_sigmoid(np.full_like(x, -40.0), x), x, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------------------
# Exponentially gated scans, gate = exp(stored logarithm) (oracle functions *_exp)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 2, 9, 64])
@pytest.mark.parametrize("with_initial", [False, True])
def test_exp_vs_autograd_of_loop(T, with_initial):
    gen = torch.Generator().manual_seed(450 + T)
    log_gates = -torch.rand(2, 2, T, generator=gen) * 2.0 + 0.3  # a few gates above 1 as well
    tokens, grad_out = (torch.randn(2, 2, T, generator=gen) for _ in range(2))
    initial = torch.randn(2, 2, generator=gen) if with_initial else torch.zeros(2, 2)
    zw, tw, iw = (t.double().requires_grad_(True) for t in (log_gates, tokens, initial))
    out = _loop_scan_from(torch.exp(zw), tw, iw)
    dz_ref, dt_ref, di_ref = torch.autograd.grad(out, (zw, tw, iw), grad_out.double())
    init_arg = initial.numpy() if with_initial else None
    fwd = seqscan.forward_exp(log_gates.numpy(), tokens.numpy(), init_arg)
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    dz, dt, di = seqscan.backward_exp(log_gates.numpy(), fwd.astype(np.float32), grad_out.numpy(), init_arg)
    np.testing.assert_allclose(dt, dt_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(di, di_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dz, dz_ref.numpy(), rtol=1e-5, atol=1e-5)  # states rounded to fp32 before the multiply


def test_exp_vs_plain_scan_of_rounded_gates_and_closed_forms():
    gen = torch.Generator().manual_seed(23)
    log_gates = -torch.rand(3, 4, 200, generator=gen)
    tokens, grad_out = (torch.randn(3, 4, 200, generator=gen) for _ in range(2))
    gates = torch.exp(log_gates.double())
    fwd = seqscan.forward_exp(log_gates.numpy(), tokens.numpy())
    plain = seqscan.forward(gates.float().numpy(), tokens.numpy())
    np.testing.assert_allclose(fwd, plain, rtol=1e-5, atol=1e-5)  # gates rounded to fp32 on one side
    states = fwd.astype(np.float32)
    dz, dx, _ = seqscan.backward_exp(log_gates.numpy(), states, grad_out.numpy())
    dg, dx_plain = seqscan.backward(gates.float().numpy(), states, grad_out.numpy())
    np.testing.assert_allclose(dx, dx_plain, rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(dz, dg * gates.numpy(), rtol=1e-5, atol=1e-5)  # d exp(z) / dz = exp(z)
    # constant logarithm log q, unit tokens: the geometric series (1 - q^(t+1)) / (1 - q)
    T, q = 40, 0.75
    z = np.full((1, 1, T), np.log(q), np.float32)
    out = seqscan.forward_exp(z, np.ones((1, 1, T), np.float32))
    qq = np.exp(np.float64(z[0, 0, 0]))
    np.testing.assert_allclose(out[0, 0], (1 - qq ** (np.arange(T) + 1)) / (1 - qq), rtol=1e-13)
    # a single unit token at t = 0: the state is exp of the running sum of the later logarithms
    z = log_gates[:1, :1, :60].numpy()
    x = np.zeros_like(z)
    x[..., 0] = 1.0
    running = np.concatenate([[0.0], np.cumsum(z[0, 0, 1:].astype(np.float64))])
    np.testing.assert_allclose(seqscan.forward_exp(z, x)[0, 0], np.exp(running), rtol=1e-12)
    # z = 0 is a running sum, z = -800 (gate 0 in fp64) returns the tokens
    x = tokens[:1, :1, :50].numpy()
    np.testing.assert_allclose(seqscan.forward_exp(np.zeros_like(x), x), np.cumsum(x.astype(np.float64), -1), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(seqscan.forward_exp(np.full_like(x, -800.0), x), x, rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------------------
# Gated interpolation x[t] = a x[t-1] + (1 - a) v[t], a = sigmoid(z) (oracle functions *_lerp)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 2, 9, 64])
@pytest.mark.parametrize("with_initial", [False, True])
def test_lerp_vs_autograd_of_loop(T, with_initial):
    """Values and all three gradients against torch autograd through the explicit
    float64 loop written with torch.lerp (x = lerp(v, x_prev, a))."""
    gen = torch.Generator().manual_seed(900 + T)
    logits = 3.0 * torch.randn(2, 2, T, generator=gen)
    values, grad_out = (torch.randn(2, 2, T, generator=gen) for _ in range(2))
    initial = torch.randn(2, 2, generator=gen) if with_initial else torch.zeros(2, 2)
    zw, vw, iw = (t.double().requires_grad_(True) for t in (logits, values, initial))
    a = torch.sigmoid(zw)
    state, outs = iw, []
    for t in range(T):
        state = torch.lerp(vw[..., t], state, a[..., t])
        outs.append(state)
    out = torch.stack(outs, dim=-1)
    dz_ref, dv_ref, di_ref = torch.autograd.grad(out, (zw, vw, iw), grad_out.double())
    init_arg = initial.numpy() if with_initial else None
    fwd = seqscan.forward_lerp(logits.numpy(), values.numpy(), init_arg)
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    dz, dv, di = seqscan.backward_lerp(logits.numpy(), values.numpy(), fwd.astype(np.float32), grad_out.numpy(), init_arg)
    np.testing.assert_allclose(dv, dv_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(di, di_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(dz, dz_ref.numpy(), rtol=1e-5, atol=1e-5)  # states rounded to fp32 before the subtraction


def test_lerp_vs_sigmoid_scan_of_formed_tokens_and_closed_forms():
    gen = torch.Generator().manual_seed(23)
    logits = 2.0 * torch.randn(3, 4, 200, generator=gen)
    values, grad_out = (torch.randn(3, 4, 200, generator=gen) for _ in range(2))
    a = torch.sigmoid(logits.double())
    tokens = ((1 - a) * values.double())
    fwd = seqscan.forward_lerp(logits.numpy(), values.numpy())
    # the sigmoid-gated scan of the tokens (1 - a) v formed outside (rounded to fp32 on that side)
    np.testing.assert_allclose(fwd, seqscan.forward_sigmoid(logits.numpy(), tokens.float().numpy()), rtol=1e-5, atol=1e-5)
    states = fwd.astype(np.float32)
    dz, dv, _ = seqscan.backward_lerp(logits.numpy(), values.numpy(), states, grad_out.numpy())
    dz_scan, dt, _ = seqscan.backward_sigmoid(logits.numpy(), states, grad_out.numpy())
    # chain rule through tokens = (1 - a) v:  d_v = d_tokens (1 - a);  d_z = d_z(scan) - d_tokens v a (1 - a)
    np.testing.assert_allclose(dv, dt * (1 - a).numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dz, dz_scan - dt * (values.double() * a * (1 - a)).numpy(), rtol=1e-8, atol=1e-10)
    # a constant value is a fixed point: started from it, the state never moves, whatever the gates
    v = np.full((2, 3, 40), 1.75, np.float32)
    z = (3 * torch.randn(2, 3, 40, generator=gen)).numpy()
    np.testing.assert_allclose(seqscan.forward_lerp(z, v, np.full((2, 3), 1.75, np.float32)), 1.75, rtol=1e-14)
    # z = 0: every gate is 1/2; unit values from a zero state give 1 - 2^-(t+1)
    T = 30
    out = seqscan.forward_lerp(np.zeros((1, 1, T), np.float32), np.ones((1, 1, T), np.float32))
    np.testing.assert_allclose(out[0, 0], 1.0 - 0.5 ** (np.arange(T) + 1), rtol=1e-15)
    # saturated gates: z = -40 returns the values, z = +40 keeps the initial state
    x = values[:1, :1, :50].numpy()
    np.testing.assert_allclose(seqscan.forward_lerp(np.full_like(x, -40.0), x), x, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(seqscan.forward_lerp(np.full_like(x, 40.0), x, np.full((1, 1), 0.5, np.float32)), 0.5,
                               rtol=1e-12, atol=1e-12)


# ---------------------------------------------------------------------------
# Exponential gate with the input scale sqrt(1 - a^2): x[t] = a x[t-1] + sqrt(1 - a^2) v[t], a = exp(z)
# (oracle functions *_expnorm)
# ---------------------------------------------------------------------------
@pytest.mark.parametrize("T", [1, 2, 9, 64])
@pytest.mark.parametrize("with_initial", [False, True])
def test_expnorm_vs_autograd_of_loop(T, with_initial):
    """Values and all three gradients against torch autograd through the explicit
    float64 loop written with torch.exp, torch.expm1 and torch.sqrt."""
    gen = torch.Generator().manual_seed(1300 + T)
    log_gates = -torch.rand(2, 2, T, generator=gen).mul(6.0).exp().mul(1e-3)  # -1e-3 ... -0.4: gates 0.67 ... 0.999
    values, grad_out = (torch.randn(2, 2, T, generator=gen) for _ in range(2))
    initial = torch.randn(2, 2, generator=gen) if with_initial else torch.zeros(2, 2)
    zw, vw, iw = (t.double().requires_grad_(True) for t in (log_gates, values, initial))
    a = torch.exp(zw)
    b = torch.sqrt(-torch.expm1(2 * zw))
    state, outs = iw, []
    for t in range(T):
        state = a[..., t] * state + b[..., t] * vw[..., t]
        outs.append(state)
    out = torch.stack(outs, dim=-1)
    dz_ref, dv_ref, di_ref = torch.autograd.grad(out, (zw, vw, iw), grad_out.double())
    init_arg = initial.numpy() if with_initial else None
    fwd = seqscan.forward_expnorm(log_gates.numpy(), values.numpy(), init_arg)
    np.testing.assert_allclose(fwd, out.detach().numpy(), rtol=1e-12, atol=1e-12)
    dz, dv, di = seqscan.backward_expnorm(log_gates.numpy(), values.numpy(), fwd.astype(np.float32), grad_out.numpy(),
                                          init_arg)
    np.testing.assert_allclose(dv, dv_ref.numpy(), rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(di, di_ref.numpy(), rtol=1e-12, atol=1e-12)
    # states rounded to fp32 before they meet the gate; the a^2 / b term is exact on both sides
    np.testing.assert_allclose(dz, dz_ref.numpy(), rtol=1e-6, atol=1e-6 * np.abs(dz_ref.numpy()).max())


def test_expnorm_vs_exp_scan_of_formed_tokens_and_closed_forms():
    gen = torch.Generator().manual_seed(29)
    log_gates = -torch.rand(3, 4, 200, generator=gen).mul(5.0).exp().mul(2e-3)
    values, grad_out = (torch.randn(3, 4, 200, generator=gen) for _ in range(2))
    z64 = log_gates.double()
    a = torch.exp(z64)
    b = torch.sqrt(-torch.expm1(2 * z64))
    tokens = b * values.double()
    fwd = seqscan.forward_expnorm(log_gates.numpy(), values.numpy())
    # the exponentially gated scan of the tokens b v formed outside (rounded to fp32 on that side)
    np.testing.assert_allclose(fwd, seqscan.forward_exp(log_gates.numpy(), tokens.float().numpy()), rtol=1e-5, atol=1e-5)
    states = fwd.astype(np.float32)
    dz, dv, di = seqscan.backward_expnorm(log_gates.numpy(), values.numpy(), states, grad_out.numpy())
    dz_scan, dt, di_scan = seqscan.backward_exp(log_gates.numpy(), states, grad_out.numpy())
    # chain rule through tokens = b v, b = sqrt(1 - exp(2 z)):  d_v = d_tokens b;  d_z = d_z(scan) - d_tokens v a^2 / b
    np.testing.assert_allclose(dv, dt * b.numpy(), rtol=1e-10, atol=1e-12)
    np.testing.assert_allclose(dz, dz_scan - dt * (values.double() * a * a / b).numpy(), rtol=1e-8, atol=1e-9)
    np.testing.assert_allclose(di, di_scan, rtol=1e-12)
    # a = 0.6 exactly-ish (z = log 0.6 rounded to fp32): b = 0.8, so x[t] = 0.6 x[t-1] + 0.8 v[t]
    T = 25
    z = np.full((1, 1, T), np.log(0.6), np.float32)
    v = values[:1, :1, :T].numpy()
    want = np.zeros(T)
    s = 0.0
    a6 = np.exp(np.float64(z[0, 0, 0]))
    for t in range(T):
        s = a6 * s + np.sqrt(1.0 - a6 * a6) * float(v[0, 0, t])
        want[t] = s
    np.testing.assert_allclose(seqscan.forward_expnorm(z, v)[0, 0], want, rtol=1e-13)
    assert abs(np.sqrt(1.0 - a6 * a6) - 0.8) < 1e-7
    # a constant value c from a zero state tends to c b / (1 - a) = c sqrt((1 + a) / (1 - a))
    out = seqscan.forward_expnorm(np.full((1, 1, 400), np.log(0.6), np.float32), np.full((1, 1, 400), 1.5, np.float32))
    np.testing.assert_allclose(out[0, 0, -1], 1.5 * np.sqrt((1 + a6) / (1 - a6)), rtol=1e-12)
    # z = -800 (gate 0): the values themselves; z = 0 (gate 1, scale 0): the initial state stays
    x = values[:1, :1, :50].numpy()
    np.testing.assert_allclose(seqscan.forward_expnorm(np.full_like(x, -800.0), x), x, rtol=1e-12, atol=1e-12)
    np.testing.assert_allclose(seqscan.forward_expnorm(np.zeros_like(x), x, np.full((1, 1), 0.5, np.float32)), 0.5,
                               rtol=1e-12, atol=1e-12)
    # unit-variance values keep a unit-variance state (what the scale is for): stationary variance b^2 / (1 - a^2) = 1
    big = torch.randn(64, 1, 20000, generator=gen)
    out = seqscan.forward_expnorm(np.full((64, 1, 20000), -0.05, np.float32), big.numpy())
    assert abs(out[:, :, 2000:].var() - 1.0) < 0.05
