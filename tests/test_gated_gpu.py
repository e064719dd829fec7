"""GPU parity tests for scans with the gate sigmoid applied inside the kernels.

The reference takes finished gates, so it has no tests of this operator; the
truth is oracle/seqscan.c's seq_*_sigmoid_f32 (sequential fp64 loops with a
fp64 sigmoid, pinned on the CPU by tests/test_oracle.py), and the operator is
tied back to the reference's by comparing it with the unfused pair
``warp.scan(torch.sigmoid(logits), tokens)`` on the GPU.

Tolerances: as tests/test_scan_gpu.py against the fp64 loops (fp32 2e-5, bf16 /
fp16 two storage ulps, relative and scaled absolute), with the fp32 figure
doubled where noted because the kernel's sigmoid (hardware exp2 and reciprocal,
about 2 ulp) enters every gate.
"""

import numpy as np
import pytest
import torch

from oracle import seqscan

pytestmark = pytest.mark.gpu

DEVICE = "cuda"
DTYPES = [torch.float32, torch.bfloat16, torch.float16]
IDS = ["fp32", "bf16", "fp16"]
storage_ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_library():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from accelerated_scan import _abi

    _abi.load()  # raises if the HIP library is missing: no fallback exists


def _inputs(rows, T, dtype, seed, logit_mean=0.0, gate="sigmoid"):
    gen = torch.Generator().manual_seed(seed)
    logits = logit_mean + 2.0 * torch.randn(rows, T, generator=gen)
    if gate == "exp":  # logarithms of gates: mostly below zero (gates in (0, 1)), one in twenty a little above
        logits = torch.where(torch.rand(rows, T, generator=gen) < 0.05, 0.05 * logits.abs(), -logits.abs())
    logits = logits.to(dtype)
    tokens = torch.randn(rows, T, generator=gen).to(dtype)
    grad_out = torch.randn(rows, T, generator=gen).to(dtype)
    initial = (3.0 * torch.randn(rows, generator=gen)).to(dtype)
    return logits, tokens, grad_out, initial


def _offset_copy(t, shape, k):
    flat = torch.empty(t.numel() + 32, dtype=t.dtype, device=DEVICE)
    view = flat[k:k + t.numel()].view(shape)
    view.copy_(t.reshape(shape))
    return view


def _run_and_compare(rows, T, dtype, seed, what, with_initial, offsets=(0, 0, 0), logit_mean=0.0, factor=2.0,
                     gate="sigmoid"):
    """``gate``: "sigmoid" (oracle functions *_sigmoid) or "exp" (*_exp; tests/test_exp_gate_gpu.py)."""
    from accelerated_scan import _abi

    code = {"sigmoid": _abi.GATE_SIGMOID, "exp": _abi.GATE_EXP}[gate]
    truth_forward, truth_backward = {"sigmoid": (seqscan.forward_sigmoid, seqscan.backward_sigmoid),
                                     "exp": (seqscan.forward_exp, seqscan.backward_exp)}[gate]
    logits, tokens, grad_out, initial = _inputs(rows, T, dtype, seed, logit_mean, gate)
    og, ox, oo = offsets
    shape = (1, rows, T)
    z, x, d = _offset_copy(logits, shape, og), _offset_copy(tokens, shape, ox), _offset_copy(grad_out, shape, oo)
    init = initial.to(DEVICE).reshape(1, rows) if with_initial else None
    out = _offset_copy(torch.zeros_like(logits), shape, oo)
    dz, dx = _offset_copy(torch.zeros_like(logits), shape, ox), _offset_copy(torch.zeros_like(tokens), shape, oo)
    di = torch.full((1, rows), float("nan"), dtype=dtype, device=DEVICE) if with_initial else None
    _abi.forward_gated(z, x, out, code, initial=init)
    _abi.backward_gated(z, out, d, dz, dx, code, initial=init, d_initial=di)
    torch.cuda.synchronize()

    f32 = lambda t: t.float().numpy()
    init_host = f32(initial) if with_initial else None
    t_out = truth_forward(f32(logits), f32(tokens), init_host)
    states = out.reshape(rows, T).cpu()  # backward consumes the states the GPU produced
    t_dz, t_dx, t_di = truth_backward(f32(logits), f32(states), f32(grad_out), init_host)
    tol = factor * 2e-5 if dtype == torch.float32 else 2 * storage_ulp[dtype]
    pairs = [("out", out, t_out), ("d_tokens", dx, t_dx), ("d_logits", dz, t_dz)]
    if with_initial:
        pairs.append(("d_initial", di, t_di))
    for name, got, want in pairs:
        got = f32(got.reshape(want.shape).cpu())
        scale = max(1.0, float(np.abs(want).max()))
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol * scale,
                                   err_msg=f"{what} {name} rows={rows} T={T} {dtype} initial={with_initial}")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
def test_every_small_T(dtype, with_initial):
    for T in list(range(1, 41)) + [63, 64, 65, 255, 256, 257, 511, 512, 513]:
        _run_and_compare(5, T, dtype, seed=T, what="small T", with_initial=with_initial)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
@pytest.mark.parametrize("rows,T", [(700, 1024), (600, 4096), (3, 16384), (300, 65536), (7, 16392), (5, 4099),
                                    (2050, 1031), (2, 65536 + 64), (513, 20000), (1024, 3000), (513, 32768)])
def test_tile_and_wave_boundaries(dtype, with_initial, rows, T):
    _run_and_compare(rows, T, dtype, seed=rows + T, what="boundaries", with_initial=with_initial)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
@pytest.mark.parametrize("rows,T", [(100000, 1), (4099, 2), (1000, 7), (777, 33), (5000, 64), (999, 255), (301, 500)])
def test_short_rows_in_groups(dtype, with_initial, rows, T):
    _run_and_compare(rows, T, dtype, seed=rows + T, what="short rows", with_initial=with_initial)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("offsets", [(1, 1, 1), (3, 3, 3), (1, 0, 2), (1, 9, 17)],
                         ids=["same1", "same3", "mixed", "same-mod-8"])
@pytest.mark.parametrize("rows,T", [(6, 2048), (3, 40000), (2050, 1031), (4, 7), (3000, 37)])
def test_unaligned_base_pointer(dtype, offsets, rows, T):
    _run_and_compare(rows, T, dtype, seed=9, what="offset views", with_initial=True, offsets=offsets)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("rows,T", [(1, 1 << 20), (3, 300000), (64, 65536), (128, 65536 + 8), (5, 99999)])
def test_split_rows(dtype, rows, T):
    from accelerated_scan import _abi

    assert _abi.load().ascan_workspace_bytes(rows, T, _abi.dtype_code(dtype)) > 0
    _run_and_compare(rows, T, dtype, seed=rows, what="split", with_initial=True)


def _random_cases(n, seed, n_dtypes):
    """Seeded random (dtype, rows, T, offsets): short rows in groups, rows of every
    tile count, few long rows; equal offsets for all tensors in 7 of 10 cases."""
    rng = np.random.RandomState(seed)
    cases = []
    for i in range(n):
        dtype_index = int(rng.randint(n_dtypes))
        rows = int(np.exp(rng.uniform(0, np.log(3000)))) if rng.rand() < 0.7 else int(rng.randint(1, 9))
        max_T = max(2, min(200000, 6_000_000 // rows))
        T = int(np.exp(rng.uniform(0, np.log(max_T))))
        k = int(rng.randint(0, 4))
        offsets = (k, k, k) if rng.rand() < 0.7 else tuple(int(v) for v in rng.randint(0, 4, size=3))
        cases.append((i, dtype_index, rows, T, offsets))
    return cases


@pytest.mark.parametrize("case", _random_cases(60, seed=20240612, n_dtypes=len(DTYPES)),
                         ids=lambda c: f"{c[0]}-{IDS[c[1]]}-{c[2]}x{c[3]}")
def test_random_shapes_and_offsets(case):
    i, dtype_index, rows, T, offsets = case
    _run_and_compare(rows, T, DTYPES[dtype_index], seed=rows * 7919 + T, what=f"random case {case}",
                     with_initial=i % 2 == 0, offsets=offsets)


def test_long_memory_fp32():
    """Gates near one (logits around +5, memory of a few hundred steps): the
    error of the in-kernel sigmoid accumulates along the row like any rounding of
    the gates would."""
    _run_and_compare(64, 65536, torch.float32, seed=1, what="long memory", with_initial=True, logit_mean=5.0,
                     factor=5.0)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_fused_equals_unfused_through_autograd(dtype):
    """sigmoid_scan(l, x, h) against warp.scan(sigmoid(l), x, h): values and all gradients."""
    from accelerated_scan.gated import sigmoid_scan
    from accelerated_scan.warp import scan

    B, C, T = 2, 48, 30000
    logits, tokens, grad_out, initial = _inputs(B * C, T, dtype, seed=3, logit_mean=1.0)
    mk = lambda t, s: t.reshape(s).to(DEVICE).requires_grad_(True)
    z1, x1, h1 = mk(logits, (B, C, T)), mk(tokens, (B, C, T)), mk(initial, (B, C))
    z2, x2, h2 = mk(logits, (B, C, T)), mk(tokens, (B, C, T)), mk(initial, (B, C))
    d = grad_out.reshape(B, C, T).to(DEVICE)
    fused = sigmoid_scan(z1, x1, h1)
    g_fused = torch.autograd.grad(fused, (z1, x1, h1), d)
    plain = scan(torch.sigmoid(z2), x2, h2)
    g_plain = torch.autograd.grad(plain, (z2, x2, h2), d)
    # fp32: both sides round every gate once (different sigmoids); 16-bit: the unfused
    # side also rounds the gates and d_gates to storage precision
    tol = 2e-5 if dtype == torch.float32 else 4 * storage_ulp[dtype]
    for name, a, b in zip(("states", "d_logits", "d_tokens", "d_initial"), (fused,) + g_fused, (plain,) + g_plain):
        scale = max(1.0, b.float().abs().max().item())
        torch.testing.assert_close(a.float(), b.float(), rtol=tol, atol=tol * scale, msg=lambda m: f"{name}: {m}")
    # zero-start form
    torch.testing.assert_close(sigmoid_scan(z1, x1).float(), scan(torch.sigmoid(z2), x2).float(), rtol=tol, atol=tol * 10)


def test_identity_gate_is_the_plain_scan_and_errors():
    from accelerated_scan import _abi
    from accelerated_scan.gated import sigmoid_scan

    lib = _abi.load()
    rows, T = 19, 3001
    logits, tokens, grad_out, initial = _inputs(rows, T, torch.float32, seed=2)
    g, x, d, h = (t.to(DEVICE) for t in (torch.sigmoid(logits), tokens, grad_out, initial))
    stream = torch.cuda.current_stream().cuda_stream
    out0, out1 = torch.empty_like(g), torch.empty_like(g)
    _abi.check(lib.ascan_forward_from(g.data_ptr(), x.data_ptr(), h.data_ptr(), out0.data_ptr(), rows, T, 0, 0, None, 0, stream))
    _abi.check(lib.ascan_forward_gated(g.data_ptr(), x.data_ptr(), h.data_ptr(), out1.data_ptr(), rows, T, 0,
                                       _abi.GATE_IDENTITY, None, 0, stream))
    assert torch.equal(out0, out1)
    # complex dtype or an unknown activation code
    assert lib.ascan_forward_gated(g.data_ptr(), x.data_ptr(), None, out1.data_ptr(), rows, T // 2, _abi.C64,
                                   _abi.GATE_SIGMOID, None, 0, stream) == 6
    assert lib.ascan_backward_gated(g.data_ptr(), out0.data_ptr(), None, d.data_ptr(), out1.data_ptr(), out1.data_ptr(),
                                    None, rows, T, 0, 7, None, 0, stream) == 6
    with pytest.raises(RuntimeError, match="activation"):
        _abi.check(6)
    with pytest.raises(RuntimeError, match="unsupported tensor dtypes"):
        sigmoid_scan(torch.polar(g, g).reshape(1, rows, T), x.reshape(1, rows, T))
    with pytest.raises(RuntimeError, match="initial"):
        sigmoid_scan(g.reshape(1, rows, T), x.reshape(1, rows, T), torch.zeros(1, rows + 1, device=DEVICE))


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_sigmoid_scan_matches_eager(backend):
    from accelerated_scan import _ops
    from accelerated_scan.gated import sigmoid_scan

    logits, tokens, grad_out, initial = _inputs(48, 3000, torch.float32, seed=77)
    z = logits.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    x = tokens.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    h = initial.reshape(2, 24).to(DEVICE).requires_grad_(True)
    w = grad_out.reshape(2, 24, 3000).to(DEVICE)
    torch.library.opcheck(_ops.scan_forward_gated, (z.detach(), x.detach(), h.detach(), 1))
    states = _ops.scan_forward_gated(z.detach(), x.detach(), h.detach(), 1)
    torch.library.opcheck(_ops.scan_backward_gated, (z.detach(), states, h.detach(), w, 1))

    def loss_fn(z, x, h, w):
        return (sigmoid_scan(z * 0.5, x, h) * w).sum()

    eager = torch.autograd.grad(loss_fn(z, x, h, w), (z, x, h))
    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    got = torch.autograd.grad(compiled(z, x, h, w), (z, x, h))
    for a, b in zip(got, eager):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
