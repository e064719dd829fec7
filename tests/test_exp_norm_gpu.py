"""GPU parity tests for the exponential gate with its variance-preserving input scale,
``x[t] = a[t] x[t-1] + sqrt(1 - a[t]^2) v[t]``, ``a = exp(z)``, ``z < 0`` -- the update of
RG-LRU / Hawk-style layers -- with gate, scale and token all formed inside the kernels.

The reference takes finished gates and tokens, so it has no tests of this
operator; the truth is oracle/seqscan.c's seq_*_expnorm_f32 (sequential fp64 loops,
pinned on the CPU by tests/test_oracle.py), and the operator is tied back to the
reference's by comparing it with the unfused sequence
``warp.scan(exp(z), sqrt(-expm1(2 z)) * v)`` on the GPU.

Tolerances as tests/test_lerp_gpu.py: fp32 4e-5 (the in-kernel exponential and square
root enter every gate and every token), bf16 / fp16 two storage ulps, relative and
scaled absolute.
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


def _inputs(rows, T, dtype, seed, logit_mean=0.0):
    """Logarithms of the gates: -exp(U(log 1e-3, log 3)) * exp(logit_mean), i.e. gates between
    0.05 and 0.999 for logit_mean = 0; more negative logit_mean moves them towards 1."""
    gen = torch.Generator().manual_seed(seed)
    spread = torch.rand(rows, T, generator=gen) * (np.log(3.0) - np.log(1e-3)) + np.log(1e-3)
    logits = (-torch.exp(spread + logit_mean)).to(dtype)
    values = torch.randn(rows, T, generator=gen).to(dtype)
    grad_out = torch.randn(rows, T, generator=gen).to(dtype)
    initial = (3.0 * torch.randn(rows, generator=gen)).to(dtype)
    return logits, values, grad_out, initial


def _offset_copy(t, shape, k):
    flat = torch.empty(t.numel() + 32, dtype=t.dtype, device=DEVICE)
    view = flat[k:k + t.numel()].view(shape)
    view.copy_(t.reshape(shape))
    return view


def _run_and_compare(rows, T, dtype, seed, what, with_initial, offsets=(0, 0, 0), logit_mean=0.0, factor=2.0):
    from accelerated_scan import _abi

    logits, values, grad_out, initial = _inputs(rows, T, dtype, seed, logit_mean)
    og, ox, oo = offsets
    shape = (1, rows, T)
    z, v, d = _offset_copy(logits, shape, og), _offset_copy(values, shape, ox), _offset_copy(grad_out, shape, oo)
    init = initial.to(DEVICE).reshape(1, rows) if with_initial else None
    out = _offset_copy(torch.zeros_like(logits), shape, oo)
    dz, dv = _offset_copy(torch.zeros_like(logits), shape, ox), _offset_copy(torch.zeros_like(values), shape, oo)
    di = torch.full((1, rows), float("nan"), dtype=dtype, device=DEVICE) if with_initial else None
    _abi.forward_gated(z, v, out, _abi.GATE_EXP_NORM, initial=init)
    _abi.backward_gated_values(z, v, out, d, dz, dv, _abi.GATE_EXP_NORM, initial=init, d_initial=di)
    torch.cuda.synchronize()

    f32 = lambda t: t.float().numpy()
    init_host = f32(initial) if with_initial else None
    t_out = seqscan.forward_expnorm(f32(logits), f32(values), init_host)
    states = out.reshape(rows, T).cpu()  # backward consumes the states the GPU produced
    t_dz, t_dv, t_di = seqscan.backward_expnorm(f32(logits), f32(values), f32(states), f32(grad_out), init_host)
    tol = factor * 2e-5 if dtype == torch.float32 else 2 * storage_ulp[dtype]
    pairs = [("out", out, t_out), ("d_values", dv, t_dv), ("d_logits", dz, t_dz)]
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
                                    (2050, 1031), (2, 65536 + 64), (513, 20000), (1024, 3000), (600, 8192)])
def test_tile_and_wave_boundaries(dtype, with_initial, rows, T):
    _run_and_compare(rows, T, dtype, seed=rows + T, what="boundaries", with_initial=with_initial)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
@pytest.mark.parametrize("rows,T", [(100000, 1), (4099, 2), (1000, 7), (777, 33), (5000, 64), (999, 255), (301, 500),
                                    (40000, 300)])
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


@pytest.mark.parametrize("dtype,rows,T", [(torch.float32, 4096, 8192), (torch.float32, 4100, 10000),
                                          (torch.bfloat16, 8192, 16384)],
                         ids=["fp32-4096x8192", "fp32-4100x10000", "bf16-8192x16384"])
def test_short_rows_of_a_large_launch_are_swept_backward(dtype, rows, T):
    """Rows of 32 to 64 KiB in tensors of 128 MiB and more (256 MiB in 16-bit storage): the backward kernel,
    whose tiles are 32 KiB, takes them by ticket instead of one workgroup per row."""
    from accelerated_scan import _abi

    assert _abi.load().ascan_workspace_bytes(rows, T, _abi.dtype_code(dtype)) > 0
    _run_and_compare(rows, T, dtype, seed=rows + T, what="short rows swept", with_initial=True)


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


@pytest.mark.parametrize("case", _random_cases(60, seed=20250923, n_dtypes=len(DTYPES)),
                         ids=lambda c: f"{c[0]}-{IDS[c[1]]}-{c[2]}x{c[3]}")
def test_random_shapes_and_offsets(case):
    i, dtype_index, rows, T, offsets = case
    _run_and_compare(rows, T, DTYPES[dtype_index], seed=rows * 7919 + T, what=f"random case {case}",
                     with_initial=i % 2 == 0, offsets=offsets)


def test_long_memory_and_short_memory_fp32():
    """Gates within 1e-5 of one (logarithms around -1e-5): 1 - gate^2 is about 2e-5 and must keep its
    relative accuracy (it is summed as a series in the logarithm, not formed as a difference); and gates
    close to zero, where the scale is 1."""
    _run_and_compare(64, 65536, torch.float32, seed=1, what="long memory", with_initial=True, logit_mean=-5.0,
                     factor=5.0)
    _run_and_compare(16, 5000, torch.float32, seed=2, what="very long memory", with_initial=True, logit_mean=-9.0,
                     factor=5.0)
    _run_and_compare(16, 5000, torch.float32, seed=3, what="short memory", with_initial=True, logit_mean=3.0)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_log_gates_at_and_next_to_zero_give_finite_gradients(dtype):
    """A stored logarithm of +0 or -0 (a 16-bit logarithm that underflowed, a layer that clamps at 0)
    makes the input scale exactly 0, where its derivative is unbounded: the backward kernel takes that
    derivative as 0, so all gradients stay finite; at the smallest negative values of the storage type
    the scale is tiny but positive and the gradients are large and finite."""
    from accelerated_scan import gated

    tiny = torch.finfo(dtype).tiny
    smallest = tiny * torch.finfo(dtype).eps  # the smallest subnormal
    T = 96
    z = torch.full((1, 3, T), -0.01, dtype=dtype)
    z[0, 0, 5], z[0, 0, 17], z[0, 0, 40], z[0, 0, 41] = 0.0, -0.0, -smallest, -tiny
    z[0, 1, :] = -0.0
    z[0, 2, ::2] = -smallest
    v = torch.randn(1, 3, T, generator=torch.Generator().manual_seed(5)).to(dtype)
    zd, vd = z.to(DEVICE).requires_grad_(), v.to(DEVICE).requires_grad_()
    out = gated.exp_norm_scan(zd, vd)
    (out.float().sum() * 1e-3).backward()  # (a small loss scale: next to zero the slope is in the thousands, and fp16 ends at 65504)
    assert torch.isfinite(out).all()
    assert torch.isfinite(zd.grad).all() and torch.isfinite(vd.grad).all()
    # a gate of exactly 1 lets no value in and passes the state on
    assert torch.equal(out[0, 1], torch.zeros_like(out[0, 1]))
    assert vd.grad[0, 1].abs().max().item() == 0.0


def test_unit_variance_values_keep_a_unit_variance_state():
    """What the scale is for: with independent unit-variance values the stationary variance of the state is
    b^2 / (1 - a^2) = 1 for every decay."""
    from accelerated_scan.gated import exp_norm_scan

    gen = torch.Generator().manual_seed(5)
    v = torch.randn(4, 64, 30000, generator=gen).to(DEVICE)
    for log_gate in (-0.5, -0.05, -0.005):
        z = torch.full_like(v, log_gate)
        out = exp_norm_scan(z, v)
        var = out[..., 5000:].var().item()
        assert abs(var - 1.0) < 0.05, (log_gate, var)


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_fused_equals_unfused_through_autograd(dtype):
    """exp_norm_scan(z, v, h) against warp.scan(exp(z), sqrt(-expm1(2 z)) * v, h): values and all gradients.
    The unfused sequence runs in fp32 on the same (stored) inputs: with 16-bit gates it would lose the
    memory that 16-bit logarithms keep, which is the reason to hand over logarithms in the first place."""
    from accelerated_scan.gated import exp_norm_scan
    from accelerated_scan.warp import scan

    B, C, T = 2, 48, 30000
    logits, values, grad_out, initial = _inputs(B * C, T, dtype, seed=3)
    mk = lambda t, s: t.reshape(s).to(DEVICE).requires_grad_(True)
    z1, v1, h1 = mk(logits, (B, C, T)), mk(values, (B, C, T)), mk(initial, (B, C))
    z2, v2, h2 = mk(logits.float(), (B, C, T)), mk(values.float(), (B, C, T)), mk(initial.float(), (B, C))
    d = grad_out.reshape(B, C, T).to(DEVICE)
    fused = exp_norm_scan(z1, v1, h1)
    g_fused = torch.autograd.grad(fused, (z1, v1, h1), d)
    a = torch.exp(z2)
    b = torch.sqrt(-torch.expm1(2 * z2))
    plain = scan(a, b * v2, h2)
    g_plain = torch.autograd.grad(plain, (z2, v2, h2), d.float())
    # 16-bit: states are stored (and read back by the backward pass) in storage precision
    tol = 4e-5 if dtype == torch.float32 else 4 * storage_ulp[dtype]
    for name, x, y in zip(("states", "d_log_gates", "d_values", "d_initial"), (fused,) + g_fused, (plain,) + g_plain):
        assert x.dtype == dtype
        scale = max(1.0, y.abs().max().item())
        torch.testing.assert_close(x.float(), y, rtol=tol, atol=tol * scale, msg=lambda m: f"{name}: {m}")
    # zero-start form
    torch.testing.assert_close(exp_norm_scan(z1, v1).float(), scan(a, b * v2), rtol=tol, atol=tol * 10)


def test_status_codes_and_validation():
    from accelerated_scan import _abi
    from accelerated_scan.gated import exp_norm_scan

    lib = _abi.load()
    rows, T = 19, 3001
    logits, values, grad_out, initial = _inputs(rows, T, torch.float32, seed=2)
    z, v, d = (t.to(DEVICE) for t in (logits, values, grad_out))
    out, dz, dv = torch.empty_like(z), torch.empty_like(z), torch.empty_like(z)
    stream = torch.cuda.current_stream().cuda_stream
    G = _abi.GATE_EXP_NORM
    # the gated backward entry point has no values argument: gates with values are refused there
    assert lib.ascan_backward_gated(z.data_ptr(), out.data_ptr(), None, d.data_ptr(), dz.data_ptr(), dv.data_ptr(),
                                    None, rows, T, 0, G, None, 0, stream) == 6
    # a gate without values; complex dtype; missing values; an output that is the values tensor
    for gate in (_abi.GATE_IDENTITY, _abi.GATE_SIGMOID, _abi.GATE_EXP, 5, -1):
        assert lib.ascan_backward_gated_values(z.data_ptr(), v.data_ptr(), out.data_ptr(), None, d.data_ptr(),
                                               dz.data_ptr(), dv.data_ptr(), None, rows, T, 0, gate, None, 0,
                                               stream) == 6
    assert lib.ascan_backward_gated_values(z.data_ptr(), v.data_ptr(), out.data_ptr(), None, d.data_ptr(),
                                           dz.data_ptr(), dv.data_ptr(), None, rows, T // 2, _abi.C64, G, None, 0,
                                           stream) == 6
    assert lib.ascan_backward_gated_values(z.data_ptr(), None, out.data_ptr(), None, d.data_ptr(), dz.data_ptr(),
                                           dv.data_ptr(), None, rows, T, 0, G, None, 0, stream) == 1
    assert lib.ascan_backward_gated_values(z.data_ptr(), v.data_ptr(), out.data_ptr(), None, d.data_ptr(),
                                           dz.data_ptr(), v.data_ptr(), None, rows, T, 0, G, None, 0, stream) == 7
    assert lib.ascan_forward_gated(z.data_ptr(), v.data_ptr(), None, out.data_ptr(), rows, T // 2, _abi.C64, G,
                                   None, 0, stream) == 6
    # the interpolating gate through the general entry point is ascan_backward_lerp, bit for bit
    _abi.forward_gated(z.reshape(1, rows, T), v.reshape(1, rows, T), out.reshape(1, rows, T), _abi.GATE_SIGMOID_LERP)
    dz2, dv2 = torch.empty_like(z), torch.empty_like(z)
    _abi.backward_lerp(z, v, out, d, dz, dv)
    _abi.backward_gated_values(z, v, out, d, dz2, dv2, _abi.GATE_SIGMOID_LERP)
    assert torch.equal(dz, dz2) and torch.equal(dv, dv2)
    with pytest.raises(RuntimeError, match="unsupported tensor dtypes"):
        exp_norm_scan(torch.polar(z.abs(), z).reshape(1, rows, T), v.reshape(1, rows, T))
    with pytest.raises(RuntimeError, match="initial"):
        exp_norm_scan(z.reshape(1, rows, T), v.reshape(1, rows, T), torch.zeros(1, rows + 1, device=DEVICE))
    # empty sequence: nothing to do, gradient of the initial state stays zero
    e = torch.empty(2, 3, 0, device=DEVICE, requires_grad=True)
    h = torch.ones(2, 3, device=DEVICE, requires_grad=True)
    assert exp_norm_scan(e, e, h).shape == (2, 3, 0)
    # a logarithm of exactly zero is gate 1 with scale 0: the state passes through, the values do not enter
    zero = torch.zeros(1, 4, 300, device=DEVICE)
    keep = exp_norm_scan(zero, torch.randn(1, 4, 300, device=DEVICE), torch.full((1, 4), 2.5, device=DEVICE))
    assert torch.equal(keep, torch.full_like(keep, 2.5))


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_exp_norm_scan_matches_eager_and_oracle(backend):
    from accelerated_scan import _abi, _ops
    from accelerated_scan.gated import exp_norm_scan

    logits, values, grad_out, initial = _inputs(48, 3000, torch.float32, seed=78)
    z = logits.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    v = values.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    h = initial.reshape(2, 24).to(DEVICE).requires_grad_(True)
    w = grad_out.reshape(2, 24, 3000).to(DEVICE)
    torch.library.opcheck(_ops.scan_forward_gated, (z.detach(), v.detach(), h.detach(), _abi.GATE_EXP_NORM))
    torch.library.opcheck(_ops.scan_forward_gated, (z, v, h, _abi.GATE_EXP_NORM))  # with its autograd formula
    states = _ops.scan_forward_gated(z.detach(), v.detach(), h.detach(), _abi.GATE_EXP_NORM)
    torch.library.opcheck(_ops.scan_backward_gated_values, (z.detach(), v.detach(), states, h.detach(), w, _abi.GATE_EXP_NORM))

    def loss_fn(z, v, h, w):
        return (exp_norm_scan(z, v, h) * w).sum()

    eager = torch.autograd.grad(loss_fn(z, v, h, w), (z, v, h))
    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    got = torch.autograd.grad(compiled(z, v, h, w), (z, v, h))
    for a, b in zip(got, eager):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
    # against the fp64 loops
    t_out = seqscan.forward_expnorm(logits.numpy(), values.numpy(), initial.numpy())
    t_dz, t_dv, t_di = seqscan.backward_expnorm(logits.numpy(), values.numpy(), states.reshape(48, 3000).cpu().numpy(),
                                             grad_out.numpy(), initial.numpy())
    np.testing.assert_allclose(states.reshape(48, 3000).cpu().numpy(), t_out, rtol=4e-5, atol=4e-5 * np.abs(t_out).max())
    for a, want in zip(got, (t_dz, t_dv, t_di)):
        np.testing.assert_allclose(a.detach().reshape(want.shape).cpu().numpy(), want, rtol=4e-5,
                                   atol=4e-5 * max(1.0, np.abs(want).max()))
    # the standalone operator is differentiable without the autograd.Function
    out = torch.ops.accelerated_scan.scan_forward_gated(z, v, h, _abi.GATE_EXP_NORM)
    alone = torch.autograd.grad((out * w).sum(), (z, v, h))
    for a, b in zip(alone, eager):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-6)
