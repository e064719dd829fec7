"""GPU parity tests for scans that start from a given state.

The reference has no such operator (its scans start from zero), so there are no
reference tests to mirror; the oracle functions seqscan.forward_from /
backward_from (sequential fp64 loops, pinned on the CPU by tests/test_oracle.py)
are the truth, together with the identity that ties the operator back to the
zero-start scan: a sequence scanned in chunks, each chunk started from the last
state of the one before, gives the states and gradients of the uncut scan.

Tolerances are those of tests/test_scan_gpu.py for comparisons with the fp64
loops: 2e-5 (relative, and absolute scaled by the largest magnitude) for fp32
and complex64, two storage ulps for bf16 / fp16.
"""

import math

import numpy as np
import pytest
import torch

from oracle import seqscan

pytestmark = pytest.mark.gpu

DEVICE = "cuda"
C64_REAL_TOKENS = "complex64 gates, float32 tokens"
ALL_DTYPES = [torch.float32, torch.bfloat16, torch.float16, torch.complex64, C64_REAL_TOKENS]
ALL_IDS = ["fp32", "bf16", "fp16", "c64", "c64_real_tokens"]
storage_ulp = {torch.bfloat16: 2.0**-8, torch.float16: 2.0**-11}


@pytest.fixture(scope="module", autouse=True)
def _need_gpu_and_library():
    assert torch.cuda.is_available(), "these tests need the MI355X"
    from accelerated_scan import _abi

    _abi.load()  # raises if the HIP library is missing: no fallback exists


def _inputs(rows, T, dtype, seed):
    """Host tensors (gates, tokens, grad_out, initial) of shape (rows, T) / (rows,)."""
    gen = torch.Generator().manual_seed(seed)
    if dtype == torch.complex64 or dtype == C64_REAL_TOKENS:
        gates = torch.polar(0.5 + 0.5 * torch.rand(rows, T, generator=gen), 2 * math.pi * torch.rand(rows, T, generator=gen))
        mk = lambda *s: torch.complex(torch.randn(*s, generator=gen), torch.randn(*s, generator=gen))
        tokens = mk(rows, T) if dtype == torch.complex64 else torch.randn(rows, T, generator=gen)
        return gates, tokens, mk(rows, T), 3.0 * mk(rows)
    gates = torch.rand(rows, T, generator=gen).to(dtype)
    tokens = torch.randn(rows, T, generator=gen).to(dtype)
    grad_out = torch.randn(rows, T, generator=gen).to(dtype)
    initial = (3.0 * torch.randn(rows, generator=gen)).to(dtype)
    return gates, tokens, grad_out, initial


def _np32(t):
    return t.numpy() if t.dtype == torch.complex64 else t.float().numpy()


def _tolerance(dtype):
    if dtype in (torch.complex64, torch.float32, C64_REAL_TOKENS):
        return 2e-5
    return 2 * storage_ulp[dtype]


def _compare(gates, tokens, grad_out, initial, out, rev, dg, dx, di, dtype, what, reverse_grads=None):
    rows, T = gates.shape
    tol = _tolerance(dtype)
    tok = _np32(tokens).astype(np.complex64) if dtype == C64_REAL_TOKENS else _np32(tokens)
    t_out = seqscan.forward_from(_np32(gates), tok, _np32(initial))
    t_rev = seqscan.forward_from(_np32(gates), tok, _np32(initial), reverse=True)
    states = out.reshape(rows, T).cpu()  # backward consumes the states the GPU produced
    t_dg, t_dx, t_di = seqscan.backward_from(_np32(gates), _np32(states), _np32(initial), _np32(grad_out))
    if dtype == C64_REAL_TOKENS:
        t_dx = t_dx.real
        assert dx.dtype == torch.float32
    pairs = [("out", out, t_out), ("rev", rev, t_rev), ("d_tokens", dx, t_dx), ("d_gates", dg, t_dg),
             ("d_initial", di, t_di)]
    if reverse_grads is not None:  # backward pass of the reverse scan, from the reverse states the GPU produced
        rdg, rdx, rdi = reverse_grads
        rev_states = rev.reshape(rows, T).cpu()
        t_rdg, t_rdx, t_rdi = seqscan.backward_from(_np32(gates), _np32(rev_states), _np32(initial), _np32(grad_out),
                                                    reverse=True)
        if dtype == C64_REAL_TOKENS:
            t_rdx = t_rdx.real
            assert rdx.dtype == torch.float32
        pairs += [("reverse d_tokens", rdx, t_rdx), ("reverse d_gates", rdg, t_rdg), ("reverse d_initial", rdi, t_rdi)]
    for name, got, want in pairs:
        got = _np32(got.reshape(want.shape).cpu())
        scale = max(1.0, float(np.abs(want).max()))
        np.testing.assert_allclose(got, want, rtol=tol, atol=tol * scale,
                                   err_msg=f"{what} {name} rows={rows} T={T} {dtype}")


def _offset_copy(t, shape, k):
    """Device copy of host tensor t whose storage starts k elements off the allocation."""
    flat = torch.empty(t.numel() + 32, dtype=t.dtype, device=DEVICE)
    view = flat[k:k + t.numel()].view(shape)
    view.copy_(t.reshape(shape))
    return view


def _run_and_compare(rows, T, dtype, seed, what, offsets=(0, 0, 0)):
    from accelerated_scan import _abi

    gates, tokens, grad_out, initial = _inputs(rows, T, dtype, seed)
    og, ox, oo = offsets
    shape = (1, rows, T)
    g, x, d = _offset_copy(gates, shape, og), _offset_copy(tokens, shape, ox), _offset_copy(grad_out, shape, oo)
    init = _offset_copy(initial, (1, rows), 1)  # one state per row; only element alignment is required
    out, rev = _offset_copy(torch.zeros_like(gates), shape, oo), _offset_copy(torch.zeros_like(gates), shape, og)
    dg, dx = _offset_copy(torch.zeros_like(gates), shape, ox), _offset_copy(torch.zeros_like(tokens), shape, oo)
    di = _offset_copy(torch.full_like(initial, float("nan")), (1, rows), 3)
    _abi.forward(g, x, out, False, initial=init)
    _abi.forward(g, x, rev, True, initial=init)
    _abi.backward(g, out, d, dg, dx, initial=init, d_initial=di)
    rdg, rdx = _offset_copy(torch.zeros_like(gates), shape, ox), _offset_copy(torch.zeros_like(tokens), shape, oo)
    rdi = _offset_copy(torch.full_like(initial, float("nan")), (1, rows), 2)
    _abi.backward(g, rev, d, rdg, rdx, initial=init, d_initial=rdi, reverse=True)
    torch.cuda.synchronize()
    _compare(gates, tokens, grad_out, initial, out, rev, dg, dx, di, dtype, what, reverse_grads=(rdg, rdx, rdi))


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=ALL_IDS)
def test_every_small_T(dtype):
    for T in list(range(1, 41)) + [63, 64, 65, 255, 256, 257, 511, 512, 513]:
        _run_and_compare(5, T, dtype, seed=T, what="small T")


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=ALL_IDS)
@pytest.mark.parametrize("rows,T", [(700, 1024), (600, 4096), (3, 16384), (300, 65536), (7, 16392), (5, 4099),
                                    (2050, 1031), (2, 65536 + 64), (513, 20000), (1024, 3000)])
def test_tile_and_wave_boundaries(dtype, rows, T):
    _run_and_compare(rows, T, dtype, seed=rows + T, what="boundaries")


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=ALL_IDS)
@pytest.mark.parametrize("rows,T", [(100000, 1), (4099, 2), (3001, 3), (1000, 7), (777, 33), (5000, 64), (1234, 100),
                                    (999, 255), (640, 256), (2, 200), (301, 500)])
def test_short_rows_in_groups(dtype, rows, T):
    """Short rows scanned in groups: every row takes its own initial state at its
    cut and returns the gradient of it."""
    _run_and_compare(rows, T, dtype, seed=rows + T, what="short rows")


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=ALL_IDS)
@pytest.mark.parametrize("offsets", [(1, 1, 1), (3, 3, 3), (1, 0, 2), (1, 9, 17), (4, 12, 8)],
                         ids=["same1", "same3", "mixed", "same-mod-8", "multiples-of-4"])
@pytest.mark.parametrize("rows,T", [(6, 2048), (3, 40000), (2050, 1031), (4, 7), (3000, 37)])
def test_unaligned_base_pointer(dtype, offsets, rows, T):
    _run_and_compare(rows, T, dtype, seed=9, what="offset views", offsets=offsets)


@pytest.mark.parametrize("dtype", ALL_DTYPES, ids=ALL_IDS)
@pytest.mark.parametrize("rows,T", [(1, 1 << 20), (3, 300000), (64, 65536), (128, 65536 + 8), (5, 99999)])
def test_split_rows(dtype, rows, T):
    """Few rows, long sequences: the tiles of a row are spread over workgroups."""
    from accelerated_scan import _abi

    code = _abi.dtype_code(torch.complex64 if dtype == C64_REAL_TOKENS else dtype,
                           torch.float32 if dtype == C64_REAL_TOKENS else None)
    assert _abi.load().ascan_workspace_bytes(rows, T, code) > 0
    _run_and_compare(rows, T, dtype, seed=rows, what="split")


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


@pytest.mark.parametrize("case", _random_cases(60, seed=20240611, n_dtypes=len(ALL_DTYPES)),
                         ids=lambda c: f"{c[0]}-{ALL_IDS[c[1]]}-{c[2]}x{c[3]}")
def test_random_shapes_and_offsets(case):
    _, dtype_index, rows, T, offsets = case
    _run_and_compare(rows, T, ALL_DTYPES[dtype_index], seed=rows * 7919 + T, what=f"random case {case}", offsets=offsets)


def test_null_initial_and_null_gradient_through_the_c_abi():
    """ascan_*_from with initial == NULL is the zero-start scan; d_initial == NULL is allowed."""
    from accelerated_scan import _abi

    lib = _abi.load()
    rows, T = 37, 5000
    gates, tokens, grad_out, initial = _inputs(rows, T, torch.float32, seed=1)
    g, x, d, init = (t.to(DEVICE) for t in (gates, tokens, grad_out, initial))
    stream = torch.cuda.current_stream().cuda_stream
    out0, out1 = torch.empty_like(g), torch.empty_like(g)
    _abi.check(lib.ascan_forward(g.data_ptr(), x.data_ptr(), out0.data_ptr(), rows, T, 0, 0, stream))
    _abi.check(lib.ascan_forward_from(g.data_ptr(), x.data_ptr(), None, out1.data_ptr(), rows, T, 0, 0, None, 0, stream))
    assert torch.equal(out0, out1)
    dg0, dx0, dg1, dx1, dg2, dx2 = (torch.empty_like(g) for _ in range(6))
    di = torch.empty_like(init)
    _abi.check(lib.ascan_backward(g.data_ptr(), out0.data_ptr(), d.data_ptr(), dg0.data_ptr(), dx0.data_ptr(), rows, T, 0, stream))
    _abi.check(lib.ascan_backward_from(g.data_ptr(), out0.data_ptr(), None, d.data_ptr(), dg1.data_ptr(), dx1.data_ptr(),
                                       di.data_ptr(), rows, T, 0, None, 0, stream))
    assert torch.equal(dg0, dg1) and torch.equal(dx0, dx1)
    torch.testing.assert_close(di, g[:, 0] * dx0[:, 0], rtol=1e-6, atol=1e-7)
    # initial given, gradient of it not wanted
    _abi.check(lib.ascan_backward_from(g.data_ptr(), out0.data_ptr(), init.data_ptr(), d.data_ptr(), dg2.data_ptr(),
                                       dx2.data_ptr(), None, rows, T, 0, None, 0, stream))
    assert torch.equal(dx2, dx0) and torch.equal(dg2[:, 1:], dg0[:, 1:])
    torch.testing.assert_close(dg2[:, 0], dx0[:, 0] * init, rtol=1e-6, atol=1e-7)


def _chunked(scan, gates, tokens, initial, cuts):
    """Scan in chunks through the autograd API, handing the last state over."""
    parts, state, begin = [], initial, 0
    for end in cuts + [gates.shape[-1]]:
        part = scan(gates[..., begin:end].contiguous(), tokens[..., begin:end].contiguous(), state)
        parts.append(part)
        state = part[..., -1]
        begin = end
    return torch.cat(parts, dim=-1)


@pytest.mark.parametrize("module,dtype", [("warp", torch.float32), ("scalar", torch.float32), ("warp", torch.bfloat16),
                                          ("complex", torch.complex64), ("complex", C64_REAL_TOKENS)],
                         ids=["warp-fp32", "scalar-fp32", "warp-bf16", "complex", "complex-real-inputs"])
def test_chunked_scan_equals_whole_scan(module, dtype):
    """Values and gradients, through autograd and d_initial, at a size where
    every chunk is many tiles long; the first chunk starts from a zero state and
    is compared with the module's two-argument scan."""
    import importlib

    scan = importlib.import_module(f"accelerated_scan.{module}").scan
    B, C, T = 2, 96, 50000
    cuts = [1, 4097, 20000, 20001, 36384]
    gates, tokens, grad_out, _ = _inputs(B * C, T, dtype, seed=5)
    if not gates.is_complex():
        gates = (0.9 + 0.1 * gates.float()).to(gates.dtype)  # long memory: the carried state matters
    g = gates.reshape(B, C, T).to(DEVICE).requires_grad_(True)
    x = tokens.reshape(B, C, T).to(DEVICE).requires_grad_(True)
    d = grad_out.reshape(B, C, T).to(DEVICE)
    zero = torch.zeros(B, C, dtype=g.dtype, device=DEVICE)

    whole = scan(g, x)
    dg_whole, dx_whole = torch.autograd.grad(whole, (g, x), d)
    parts = _chunked(scan, g, x, zero, cuts)
    dg_parts, dx_parts = torch.autograd.grad(parts, (g, x), d)

    if dtype in (torch.bfloat16,):
        # the state crosses a chunk boundary in storage precision, as it does inside the whole scan's output
        tol = dict(rtol=4 * storage_ulp[dtype], atol=4 * storage_ulp[dtype] * whole.float().abs().max().item())
    else:
        tol = dict(rtol=2e-5, atol=2e-5 * whole.abs().max().item())
    torch.testing.assert_close(parts, whole, **tol)
    gtol = dict(rtol=tol["rtol"], atol=tol["rtol"] * max(1.0, dx_whole.abs().max().item()))
    torch.testing.assert_close(dx_parts, dx_whole, **gtol)
    gtol = dict(rtol=tol["rtol"], atol=tol["rtol"] * max(1.0, dg_whole.abs().max().item()))
    torch.testing.assert_close(dg_parts, dg_whole, **gtol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.complex64, C64_REAL_TOKENS],
                         ids=["fp32", "bf16", "c64", "c64_real_tokens"])
@pytest.mark.parametrize("mode", ["eager", "aot_eager"])
def test_bidirectional_scan_through_autograd(dtype, mode):
    """A sequence scanned in both directions, ``scan(g, x, h) + scan(g, x, h, reverse=True)``, through the
    modules' autograd nodes: values and all gradients against the fp64 loops (the reverse scan has a fused
    backward kernel of its own)."""
    from accelerated_scan import stateful
    from accelerated_scan.warp import scan as warp_scan

    B, C, T = 2, 40, 20011
    gates, tokens, grad_out, initial = _inputs(B * C, T, dtype, seed=21)
    g = gates.reshape(B, C, T).to(DEVICE).requires_grad_(True)
    x = tokens.reshape(B, C, T).to(DEVICE).requires_grad_(True)
    h = initial.reshape(B, C).to(DEVICE).requires_grad_(True)
    d = grad_out.reshape(B, C, T).to(DEVICE)

    def both(g, x, h):
        return stateful.scan(g, x, h), stateful.scan(g, x, h, reverse=True)

    fn = torch.compile(both, backend=mode, fullgraph=True) if mode != "eager" else both
    fwd, rev = fn(g, x, h)
    dg, dx, dh = torch.autograd.grad(fwd + rev, (g, x, h), d)

    tol = _tolerance(dtype)
    G, X, H, D = _np32(gates), _np32(tokens), _np32(initial), _np32(grad_out)
    tok = X.astype(np.complex64) if dtype == C64_REAL_TOKENS else X
    t_fwd = seqscan.forward_from(G, tok, H)
    t_rev = seqscan.forward_from(G, tok, H, reverse=True)
    f_dg, f_dx, f_dh = seqscan.backward_from(G, _np32(fwd.detach().reshape(B * C, T).cpu()), H, D)
    r_dg, r_dx, r_dh = seqscan.backward_from(G, _np32(rev.detach().reshape(B * C, T).cpu()), H, D, reverse=True)
    t_dx = f_dx + r_dx
    if dtype == C64_REAL_TOKENS:
        t_dx = t_dx.real
    # the two gradients are summed by autograd in storage precision: one more rounding for 16-bit
    gtol = tol if dtype != torch.bfloat16 else 2 * tol
    for name, got, want, t in (("forward states", fwd, t_fwd, tol), ("reverse states", rev, t_rev, tol),
                               ("d_tokens", dx, t_dx, gtol), ("d_gates", dg, f_dg + r_dg, gtol),
                               ("d_initial", dh, f_dh + r_dh, gtol)):
        got = _np32(got.detach().reshape(want.shape).cpu())
        scale = max(1.0, float(np.abs(want).max()))
        np.testing.assert_allclose(got, want, rtol=t, atol=t * scale, err_msg=f"{name} {dtype} {mode}")
    # the keyword of warp.scan / scalar.scan / complex.scan reaches the same operator
    if dtype in (torch.float32, torch.bfloat16):
        from accelerated_scan.scalar import scan as scalar_scan

        assert torch.equal(scalar_scan(g, x, h, reverse=True), rev)
        assert torch.equal(scalar_scan(g, x, reverse=True), warp_scan(g, x, reverse=True))
    else:
        from accelerated_scan.complex import scan as complex_scan

        assert torch.equal(complex_scan(g, x, h, reverse=True), rev)
        assert torch.equal(complex_scan(g, x, reverse=True), stateful.scan(g, x, None, reverse=True))
    if dtype in (torch.float32, torch.bfloat16):
        assert torch.equal(warp_scan(g, x, h, reverse=True), rev)
        torch.testing.assert_close(warp_scan(g, x, reverse=True).float(),
                                   stateful.scan(g, x, torch.zeros_like(h), reverse=True).float(), rtol=0, atol=0)


def test_gradient_of_initial_against_autograd_of_the_loop():
    from accelerated_scan.warp import scan

    B, C, T = 2, 3, 70
    gates, tokens, grad_out, initial = _inputs(B * C, T, torch.float32, seed=8)
    g, x, d = (t.reshape(B, C, T) for t in (gates, tokens, grad_out))
    i = initial.reshape(B, C)
    g64, x64, i64 = (t.double().requires_grad_(True) for t in (g, x, i))
    state, outs = i64, []
    for t in range(T):
        state = g64[..., t] * state + x64[..., t]
        outs.append(state)
    want = torch.autograd.grad(torch.stack(outs, -1), (g64, x64, i64), d.double())
    gd, xd, idev = (t.to(DEVICE).requires_grad_(True) for t in (g, x, i))
    got = torch.autograd.grad(scan(gd, xd, idev), (gd, xd, idev), d.to(DEVICE))
    for a, b in zip(got, want):
        torch.testing.assert_close(a.cpu().double(), b, rtol=2e-5, atol=2e-5)


def test_streaming_decode_one_token_at_a_time():
    """T = 1 calls carrying the state: the degenerate chunking used by token-by-token inference."""
    from accelerated_scan import stateful
    from accelerated_scan.warp import scan

    B, C, T = 2, 64, 48
    gates, tokens, _, _ = _inputs(B * C, T, torch.float32, seed=13)
    g, x = gates.reshape(B, C, T).to(DEVICE), tokens.reshape(B, C, T).to(DEVICE)
    whole = scan(g, x)
    state = torch.zeros(B, C, device=DEVICE)
    for t in range(T):
        state = stateful.scan_forward(g[..., t:t + 1].contiguous(), x[..., t:t + 1].contiguous(), state)[..., 0]
        torch.testing.assert_close(state, whole[..., t], rtol=1e-5, atol=1e-5)


def test_validation():
    from accelerated_scan.complex import scan as complex_scan
    from accelerated_scan.warp import scan

    g = torch.rand(2, 3, 16, device=DEVICE)
    x = torch.rand(2, 3, 16, device=DEVICE)
    with pytest.raises(RuntimeError, match="initial"):
        scan(g, x, torch.zeros(2, 4, device=DEVICE))
    with pytest.raises(RuntimeError, match="initial"):
        scan(g, x, torch.zeros(2, 3, device=DEVICE, dtype=torch.bfloat16))
    with pytest.raises(RuntimeError, match="device"):
        scan(g, x, torch.zeros(2, 3))
    with pytest.raises(TypeError):
        complex_scan(g, x, torch.zeros(2, 3, device=DEVICE))
    # empty sequence: no states, zero gradient for the initial state
    i = torch.ones(2, 3, device=DEVICE, requires_grad=True)
    e = scan(g[..., :0].contiguous(), x[..., :0].contiguous(), i)
    assert e.shape == (2, 3, 0)
    (di,) = torch.autograd.grad(e.sum(), (i,))
    assert torch.equal(di, torch.zeros_like(i))
