"""GPU parity tests for scans whose gates are stored as logarithms,
``x[t] = exp(log_gates[t]) * x[t-1] + tokens[t]``, with the exponential inside the
kernels (ASCAN_GATE_EXP).

The reference takes finished gates, so it has no tests of this operator; the
truth is oracle/seqscan.c's seq_*_exp_f32 (sequential fp64 loops, pinned on the
CPU by tests/test_oracle.py), and the operator is tied back to the reference's by
comparing it with ``warp.scan(exp(log_gates), tokens)`` on the GPU.  Shapes,
offsets and tolerances are those of tests/test_gated_gpu.py, whose helper runs
the cases.
"""

import numpy as np
import pytest
import torch

from oracle import seqscan
from test_gated_gpu import DEVICE, DTYPES, IDS, _inputs, _random_cases, _run_and_compare, storage_ulp

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_library():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from accelerated_scan import _abi

    _abi.load()  # raises if the HIP library is missing: no fallback exists


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
def test_every_small_T(dtype, with_initial):
    for T in list(range(1, 41)) + [63, 64, 65, 255, 256, 257, 511, 512, 513]:
        _run_and_compare(5, T, dtype, seed=T, what="small T", with_initial=with_initial, gate="exp")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("with_initial", [False, True], ids=["zero-start", "initial"])
@pytest.mark.parametrize("rows,T", [(700, 1024), (600, 4096), (3, 16384), (300, 65536), (7, 16392), (5, 4099),
                                    (2050, 1031), (2, 65536 + 64), (513, 20000), (1024, 3000), (100000, 1), (4099, 2),
                                    (1000, 7), (777, 33), (5000, 64), (999, 255), (301, 500)])
def test_boundaries_and_short_rows(dtype, with_initial, rows, T):
    _run_and_compare(rows, T, dtype, seed=rows + T, what="boundaries", with_initial=with_initial, gate="exp")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("offsets", [(1, 1, 1), (3, 3, 3), (1, 0, 2), (1, 9, 17)],
                         ids=["same1", "same3", "mixed", "same-mod-8"])
@pytest.mark.parametrize("rows,T", [(6, 2048), (3, 40000), (2050, 1031), (4, 7), (3000, 37)])
def test_unaligned_base_pointer(dtype, offsets, rows, T):
    _run_and_compare(rows, T, dtype, seed=9, what="offset views", with_initial=True, offsets=offsets, gate="exp")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
@pytest.mark.parametrize("rows,T", [(1, 1 << 20), (3, 300000), (64, 65536), (128, 65536 + 8), (5, 99999)])
def test_split_rows(dtype, rows, T):
    from accelerated_scan import _abi

    assert _abi.load().ascan_workspace_bytes(rows, T, _abi.dtype_code(dtype)) > 0
    _run_and_compare(rows, T, dtype, seed=rows, what="split", with_initial=True, gate="exp")


@pytest.mark.parametrize("case", _random_cases(40, seed=20240615, n_dtypes=len(DTYPES)),
                         ids=lambda c: f"{c[0]}-{IDS[c[1]]}-{c[2]}x{c[3]}")
def test_random_shapes_and_offsets(case):
    i, dtype_index, rows, T, offsets = case
    _run_and_compare(rows, T, DTYPES[dtype_index], seed=rows * 7919 + T, what=f"random case {case}",
                     with_initial=i % 2 == 0, offsets=offsets, gate="exp")


@pytest.mark.parametrize("dtype", DTYPES, ids=IDS)
def test_fused_equals_unfused_through_autograd(dtype):
    """exp_scan(z, x, h) against warp.scan(exp(z), x, h): values and all gradients."""
    from accelerated_scan.gated import exp_scan
    from accelerated_scan.warp import scan

    B, C, T = 2, 48, 30000
    log_gates, tokens, grad_out, initial = _inputs(B * C, T, dtype, seed=3, gate="exp")
    mk = lambda t, s: t.reshape(s).to(DEVICE).requires_grad_(True)
    z1, x1, h1 = mk(log_gates, (B, C, T)), mk(tokens, (B, C, T)), mk(initial, (B, C))
    z2, x2, h2 = mk(log_gates, (B, C, T)), mk(tokens, (B, C, T)), mk(initial, (B, C))
    d = grad_out.reshape(B, C, T).to(DEVICE)
    fused = exp_scan(z1, x1, h1)
    g_fused = torch.autograd.grad(fused, (z1, x1, h1), d)
    plain = scan(torch.exp(z2), x2, h2)
    g_plain = torch.autograd.grad(plain, (z2, x2, h2), d)
    # 16-bit: the unfused side also rounds the gates and d_gates to storage precision
    tol = 2e-5 if dtype == torch.float32 else 4 * storage_ulp[dtype]
    for name, a, b in zip(("states", "d_log_gates", "d_tokens", "d_initial"), (fused,) + g_fused, (plain,) + g_plain):
        scale = max(1.0, b.float().abs().max().item())
        torch.testing.assert_close(a.float(), b.float(), rtol=tol, atol=tol * scale, msg=lambda m: f"{name}: {m}")
    torch.testing.assert_close(exp_scan(z1, x1).float(), scan(torch.exp(z2), x2).float(), rtol=tol, atol=tol * 10)


def test_bf16_logarithms_keep_long_memory():
    """Gates 0.999..1 held in bf16: as gates they collapse to 0.99609375 or 1, as logarithms they keep three
    digits.  The states of exp_scan on bf16 logarithms stay within a few percent of the fp64 scan of the exact
    gates; warp.scan on the bf16-rounded gates is off by far more."""
    from accelerated_scan.gated import exp_scan
    from accelerated_scan.warp import scan

    gen = torch.Generator().manual_seed(5)
    rows, T = 64, 8192
    gates = 0.999 + 0.001 * torch.rand(rows, T, generator=gen, dtype=torch.float64)
    tokens = torch.rand(rows, T, generator=gen).bfloat16()
    truth = seqscan.forward(gates.float().numpy(), tokens.float().numpy())  # gates exact to fp32
    z = gates.log().bfloat16().reshape(1, rows, T).to(DEVICE)
    x = tokens.reshape(1, rows, T).to(DEVICE)
    via_logs = exp_scan(z, x).float().cpu().numpy().reshape(rows, T)
    via_gates = scan(gates.bfloat16().reshape(1, rows, T).to(DEVICE), x).float().cpu().numpy().reshape(rows, T)
    err_logs = np.abs(via_logs - truth).max() / np.abs(truth).max()
    err_gates = np.abs(via_gates - truth).max() / np.abs(truth).max()
    print(f"bf16 long memory: relative error with logarithms {err_logs:.3e}, with gates {err_gates:.3e}")
    assert err_logs <= 2e-2
    assert err_gates >= 5 * err_logs


def test_exp_gate_validation_and_compile():
    from accelerated_scan import _abi, _ops
    from accelerated_scan.gated import exp_scan

    lib = _abi.load()
    rows, T = 19, 3001
    log_gates, tokens, grad_out, initial = _inputs(rows, T, torch.float32, seed=2, gate="exp")
    z, x, d, h = (t.to(DEVICE) for t in (log_gates, tokens, grad_out, initial))
    stream = torch.cuda.current_stream().cuda_stream
    out = torch.empty_like(z)
    # complex dtype: refused
    assert lib.ascan_forward_gated(z.data_ptr(), x.data_ptr(), None, out.data_ptr(), rows, T // 2, _abi.C64,
                                   _abi.GATE_EXP, None, 0, stream) == 6
    with pytest.raises(RuntimeError, match="unsupported tensor dtypes"):
        exp_scan(torch.polar(z.exp(), z).reshape(1, rows, T), x.reshape(1, rows, T))

    z3 = z.reshape(1, rows, T).clone().requires_grad_(True)
    x3 = x.reshape(1, rows, T).clone().requires_grad_(True)
    h3 = h.reshape(1, rows).clone().requires_grad_(True)
    w = d.reshape(1, rows, T)
    torch.library.opcheck(_ops.scan_forward_gated, (z3.detach(), x3.detach(), h3.detach(), _abi.GATE_EXP))

    def loss_fn(z, x, h, w):
        return (exp_scan(z * 0.5, x, h) * w).sum()

    eager = torch.autograd.grad(loss_fn(z3, x3, h3, w), (z3, x3, h3))
    compiled = torch.compile(loss_fn, backend="aot_eager", fullgraph=True)
    got = torch.autograd.grad(compiled(z3, x3, h3, w), (z3, x3, h3))
    for a, b in zip(got, eager):
        torch.testing.assert_close(a, b, rtol=1e-5, atol=1e-5)
    # the standalone operator is differentiable too (its own autograd formula)
    states = torch.ops.accelerated_scan.scan_forward_gated(z3, x3, h3, _abi.GATE_EXP)
    direct = torch.autograd.grad(states, (z3, x3, h3), w)
    viafn = torch.autograd.grad(exp_scan(z3, x3, h3), (z3, x3, h3), w)
    for a, b in zip(direct, viafn):
        assert torch.equal(a, b)
