"""GPU parity tests for the gated interpolation
``x[t] = a[t] x[t-1] + (1 - a[t]) v[t]``, ``a = sigmoid(z)``, with gate and token
both formed inside the kernels.

The reference takes finished gates and tokens, so it has no tests of this
operator; the truth is oracle/seqscan.c's seq_*_lerp_f32 (sequential fp64 loops,
pinned on the CPU by tests/test_oracle.py), and the operator is tied back to the
reference's by comparing it with the unfused sequence
``warp.scan(sigmoid(z), (1 - sigmoid(z)) * v)`` on the GPU.

Tolerances as tests/test_gated_gpu.py: fp32 4e-5 (the in-kernel sigmoid enters
every gate and every token), bf16 / fp16 two storage ulps, relative and scaled
absolute.
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
    gen = torch.Generator().manual_seed(seed)
    logits = (logit_mean + 2.0 * torch.randn(rows, T, generator=gen)).to(dtype)
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
    _abi.forward_gated(z, v, out, _abi.GATE_SIGMOID_LERP, initial=init)
    _abi.backward_lerp(z, v, out, d, dz, dv, initial=init, d_initial=di)
    torch.cuda.synchronize()

    f32 = lambda t: t.float().numpy()
    init_host = f32(initial) if with_initial else None
    t_out = seqscan.forward_lerp(f32(logits), f32(values), init_host)
    states = out.reshape(rows, T).cpu()  # backward consumes the states the GPU produced
    t_dz, t_dv, t_di = seqscan.backward_lerp(f32(logits), f32(values), f32(states), f32(grad_out), init_host)
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


@pytest.mark.parametrize("case", _random_cases(60, seed=20250117, n_dtypes=len(DTYPES)),
                         ids=lambda c: f"{c[0]}-{IDS[c[1]]}-{c[2]}x{c[3]}")
def test_random_shapes_and_offsets(case):
    i, dtype_index, rows, T, offsets = case
    _run_and_compare(rows, T, DTYPES[dtype_index], seed=rows * 7919 + T, what=f"random case {case}",
                     with_initial=i % 2 == 0, offsets=offsets)


def test_long_memory_and_saturated_gates_fp32():
    """Gates near one (logits around +5): 1 - gate is small and must keep its
    relative accuracy (it is evaluated as sigmoid(-z), not as a difference)."""
    _run_and_compare(64, 65536, torch.float32, seed=1, what="long memory", with_initial=True, logit_mean=5.0,
                     factor=5.0)
    _run_and_compare(16, 5000, torch.float32, seed=2, what="saturated high", with_initial=True, logit_mean=14.0)
    _run_and_compare(16, 5000, torch.float32, seed=3, what="saturated low", with_initial=True, logit_mean=-14.0)


def test_constant_value_is_a_fixed_point():
    """Started from v, a row of constant values v stays at v whatever the gates do: bit for bit,
    since a + (1 - a) is exactly representable only by luck, the bar is 2 ulp."""
    from accelerated_scan.gated import sigmoid_lerp_scan

    gen = torch.Generator().manual_seed(5)
    z = (3 * torch.randn(2, 33, 9000, generator=gen)).to(DEVICE)
    v = torch.full((2, 33, 9000), 1.75, device=DEVICE)
    out = sigmoid_lerp_scan(z, v, torch.full((2, 33), 1.75, device=DEVICE))
    assert (out - 1.75).abs().max().item() <= 4 * 2.0 ** -23 * 1.75 * 10  # rounding random-walks along 9000 steps


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_fused_equals_unfused_through_autograd(dtype):
    """sigmoid_lerp_scan(z, v, h) against warp.scan(sigmoid(z), (1 - sigmoid(z)) * v, h): values and all gradients."""
    from accelerated_scan.gated import sigmoid_lerp_scan
    from accelerated_scan.warp import scan

    B, C, T = 2, 48, 30000
    logits, values, grad_out, initial = _inputs(B * C, T, dtype, seed=3, logit_mean=1.0)
    mk = lambda t, s: t.reshape(s).to(DEVICE).requires_grad_(True)
    z1, v1, h1 = mk(logits, (B, C, T)), mk(values, (B, C, T)), mk(initial, (B, C))
    z2, v2, h2 = mk(logits, (B, C, T)), mk(values, (B, C, T)), mk(initial, (B, C))
    d = grad_out.reshape(B, C, T).to(DEVICE)
    fused = sigmoid_lerp_scan(z1, v1, h1)
    g_fused = torch.autograd.grad(fused, (z1, v1, h1), d)
    a = torch.sigmoid(z2)
    plain = scan(a, (1 - a) * v2, h2)
    g_plain = torch.autograd.grad(plain, (z2, v2, h2), d)
    # 16-bit: the unfused side rounds gates, tokens and their gradients to storage precision on the way
    tol = 4e-5 if dtype == torch.float32 else 6 * storage_ulp[dtype]
    for name, x, y in zip(("states", "d_logits", "d_values", "d_initial"), (fused,) + g_fused, (plain,) + g_plain):
        scale = max(1.0, y.float().abs().max().item())
        torch.testing.assert_close(x.float(), y.float(), rtol=tol, atol=tol * scale, msg=lambda m: f"{name}: {m}")
    # zero-start form
    torch.testing.assert_close(sigmoid_lerp_scan(z1, v1).float(), scan(a, (1 - a) * v2).float(), rtol=tol, atol=tol * 10)


def test_status_codes_and_validation():
    from accelerated_scan import _abi
    from accelerated_scan.gated import sigmoid_lerp_scan

    lib = _abi.load()
    rows, T = 19, 3001
    logits, values, grad_out, initial = _inputs(rows, T, torch.float32, seed=2)
    z, v, d = (t.to(DEVICE) for t in (logits, values, grad_out))
    out, dz, dv = torch.empty_like(z), torch.empty_like(z), torch.empty_like(z)
    stream = torch.cuda.current_stream().cuda_stream
    # the gated backward entry point has no values argument: the interpolating gate is refused there
    assert lib.ascan_backward_gated(z.data_ptr(), out.data_ptr(), None, d.data_ptr(), dz.data_ptr(), dv.data_ptr(),
                                    None, rows, T, 0, _abi.GATE_SIGMOID_LERP, None, 0, stream) == 6
    # complex dtype; missing values; an output that is the values tensor
    assert lib.ascan_backward_lerp(z.data_ptr(), v.data_ptr(), out.data_ptr(), None, d.data_ptr(), dz.data_ptr(),
                                   dv.data_ptr(), None, rows, T // 2, _abi.C64, None, 0, stream) == 6
    assert lib.ascan_backward_lerp(z.data_ptr(), None, out.data_ptr(), None, d.data_ptr(), dz.data_ptr(),
                                   dv.data_ptr(), None, rows, T, 0, None, 0, stream) == 1
    assert lib.ascan_backward_lerp(z.data_ptr(), v.data_ptr(), out.data_ptr(), None, d.data_ptr(), dz.data_ptr(),
                                   v.data_ptr(), None, rows, T, 0, None, 0, stream) == 7
    assert lib.ascan_forward_gated(z.data_ptr(), v.data_ptr(), None, out.data_ptr(), rows, T // 2, _abi.C64,
                                   _abi.GATE_SIGMOID_LERP, None, 0, stream) == 6
    with pytest.raises(RuntimeError, match="unsupported tensor dtypes"):
        sigmoid_lerp_scan(torch.polar(z.abs(), z).reshape(1, rows, T), v.reshape(1, rows, T))
    with pytest.raises(RuntimeError, match="initial"):
        sigmoid_lerp_scan(z.reshape(1, rows, T), v.reshape(1, rows, T), torch.zeros(1, rows + 1, device=DEVICE))
    # empty sequence: nothing to do, gradient of the initial state stays zero
    e = torch.empty(2, 3, 0, device=DEVICE, requires_grad=True)
    h = torch.ones(2, 3, device=DEVICE, requires_grad=True)
    assert sigmoid_lerp_scan(e, e, h).shape == (2, 3, 0)


@pytest.mark.parametrize("backend", ["aot_eager", "inductor"])
def test_compiled_lerp_scan_matches_eager_and_oracle(backend):
    from accelerated_scan import _abi, _ops
    from accelerated_scan.gated import sigmoid_lerp_scan

    logits, values, grad_out, initial = _inputs(48, 3000, torch.float32, seed=78)
    z = logits.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    v = values.reshape(2, 24, 3000).to(DEVICE).requires_grad_(True)
    h = initial.reshape(2, 24).to(DEVICE).requires_grad_(True)
    w = grad_out.reshape(2, 24, 3000).to(DEVICE)
    torch.library.opcheck(_ops.scan_forward_gated, (z.detach(), v.detach(), h.detach(), _abi.GATE_SIGMOID_LERP))
    torch.library.opcheck(_ops.scan_forward_gated, (z, v, h, _abi.GATE_SIGMOID_LERP))  # with its autograd formula
    states = _ops.scan_forward_gated(z.detach(), v.detach(), h.detach(), _abi.GATE_SIGMOID_LERP)
    torch.library.opcheck(_ops.scan_backward_lerp, (z.detach(), v.detach(), states, h.detach(), w))

    def loss_fn(z, v, h, w):
        return (sigmoid_lerp_scan(z, v, h) * w).sum()

    eager = torch.autograd.grad(loss_fn(z, v, h, w), (z, v, h))
    compiled = torch.compile(loss_fn, backend=backend, fullgraph=True)
    got = torch.autograd.grad(compiled(z, v, h, w), (z, v, h))
    for a, b in zip(got, eager):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
    # against the fp64 loops
    t_out = seqscan.forward_lerp(logits.numpy(), values.numpy(), initial.numpy())
    t_dz, t_dv, t_di = seqscan.backward_lerp(logits.numpy(), values.numpy(), states.reshape(48, 3000).cpu().numpy(),
                                             grad_out.numpy(), initial.numpy())
    np.testing.assert_allclose(states.reshape(48, 3000).cpu().numpy(), t_out, rtol=4e-5, atol=4e-5 * np.abs(t_out).max())
    for a, want in zip(got, (t_dz, t_dv, t_di)):
        np.testing.assert_allclose(a.detach().reshape(want.shape).cpu().numpy(), want, rtol=4e-5,
                                   atol=4e-5 * max(1.0, np.abs(want).max()))
    # the standalone operator is differentiable without the autograd.Function
    out = torch.ops.accelerated_scan.scan_forward_gated(z, v, h, _abi.GATE_SIGMOID_LERP)
    alone = torch.autograd.grad((out * w).sum(), (z, v, h))
    for a, b in zip(alone, eager):
        torch.testing.assert_close(a, b, rtol=1e-6, atol=1e-6)
