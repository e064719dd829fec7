"""ascan_forward_split_static: the split-row forward scan with its table in the
library's static device array, for callers that cannot allocate.  Called through
the raw C ABI and compared with ascan_forward_split (caller-provided workspace)
and with the fp64 recurrence, on two calls in a row, the second one smaller, so
that the second call meets the first call's leftovers in the shared array.

A tile of a split row receives the state entering its window of 64 tiles folded
with the aggregates of the window's earlier tiles in one fixed order, so the two
entry points agree bit for bit; against the fp64 recurrence the bar is the fp32
one of the other GPU tests, 2e-5 relative to the largest magnitude.
"""

import ctypes

import numpy as np
import pytest
import torch

from oracle import seqscan

pytestmark = pytest.mark.gpu

DEVICE = "cuda"
TOO_LARGE = 8


def _inputs(rows, T, dtype, seed):
    gen = torch.Generator().manual_seed(seed)
    gates = (0.9 + 0.1 * torch.rand(rows, T, generator=gen)).to(dtype)
    tokens = torch.randn(rows, T, generator=gen).to(dtype)
    return gates, tokens


def _run_both(lib, gates, tokens, code, reverse):
    from accelerated_scan import _abi

    rows, T = gates.shape
    g, x = gates.to(DEVICE), tokens.to(DEVICE)
    nbytes = lib.ascan_workspace_bytes(rows, T, code)
    assert 0 < nbytes <= 4 * 1024 * 1024, "the case must be a split one that fits the static array"
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=DEVICE)
    want = torch.empty_like(g)
    got = torch.full_like(g, float("nan"))
    stream = torch.cuda.current_stream().cuda_stream
    _abi.check(lib.ascan_forward_split(g.data_ptr(), x.data_ptr(), want.data_ptr(), rows, T, code, int(reverse),
                                       workspace.data_ptr(), nbytes, stream))
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    _abi.check(lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), got.data_ptr(), rows, T, code,
                                              int(reverse), stream))
    torch.cuda.synchronize()
    free_after = torch.cuda.mem_get_info()[0]
    assert _abi.workspace_timeouts(workspace) == 0
    ran_out = ctypes.c_uint(99)
    _abi.check(lib.ascan_static_workspace_timeouts(ctypes.byref(ran_out), stream))
    assert ran_out.value == 0, "a wait of the call on the static table ran out"
    return got, want, free_before - free_after


def _check(got, want, gates, tokens, reverse, tol):
    truth = seqscan.forward(gates.float().numpy(), tokens.float().numpy(), reverse=reverse)
    scale = max(1.0, float(np.abs(truth).max()))
    assert torch.equal(got, want), "static table against caller-provided workspace"
    np.testing.assert_allclose(got.float().cpu().numpy(), truth, rtol=tol, atol=tol * scale,
                               err_msg="static table against the fp64 recurrence")


@pytest.mark.parametrize("dtype,code,tol", [(torch.float32, 0, 2e-5), (torch.bfloat16, 1, 2.0 ** -7)],
                         ids=["fp32", "bf16"])
def test_static_table_twice_in_a_row_second_call_smaller(dtype, code, tol):
    assert torch.cuda.is_available(), "this test needs the MI355X"
    from accelerated_scan import _abi

    lib = _abi.load()
    first = _inputs(5, 400000, dtype, seed=101)    # 5 rows x 25 or 49 tiles
    second = _inputs(2, 70001, dtype, seed=102)    # fewer rows, fewer tiles, odd length
    grown = []
    for (gates, tokens), reverse in ((first, False), (second, False), (first, True), (second, True)):
        got, want, grew = _run_both(lib, gates, tokens, code, reverse)
        _check(got, want, gates, tokens, reverse, tol)
        grown.append(grew)
    # the array exists once per GPU from the first use of the library on; later calls take no device memory
    assert all(g <= 0 for g in grown[1:]), grown


def test_static_table_limit_and_unsplit_shapes():
    from accelerated_scan import _abi

    lib = _abi.load()
    g = torch.rand(4, 256, device=DEVICE)
    x = torch.rand(4, 256, device=DEVICE)
    out = torch.empty_like(g)
    stream = torch.cuda.current_stream().cuda_stream
    # 128 rows of 2^24 elements: 128 x 2049 records of 64 bytes, more than the 4 MiB array -- refused before any access
    assert lib.ascan_workspace_bytes(128, 1 << 24, 0) > 4 * 1024 * 1024
    assert lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), out.data_ptr(), 128, 1 << 24, 0, 0, stream) == TOO_LARGE
    assert "static workspace" in lib.ascan_status_string(TOO_LARGE).decode()
    # a shape that is not split runs the plain kernels: same bits as ascan_forward
    want = torch.empty_like(g)
    _abi.check(lib.ascan_forward(g.data_ptr(), x.data_ptr(), want.data_ptr(), 4, 256, 0, 0, stream))
    _abi.check(lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), out.data_ptr(), 4, 256, 0, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    # a shape of which only the backward kernel would be swept (many complex rows of 64 KiB): ascan_workspace_bytes
    # reports a table beyond the array's size, but the forward kernel takes none, so the call is not refused
    rows, T = 24000, 8192
    assert lib.ascan_workspace_bytes(rows, T, 3) > 4 * 1024 * 1024
    cg = torch.polar(0.5 + 0.5 * torch.rand(rows, T, device=DEVICE), 6.28 * torch.rand(rows, T, device=DEVICE))
    cx = torch.randn(rows, T, device=DEVICE, dtype=torch.complex64)
    cout, cwant = torch.empty_like(cx), torch.empty_like(cx)
    _abi.check(lib.ascan_forward(cg.data_ptr(), cx.data_ptr(), cwant.data_ptr(), rows, T, 3, 0, stream))
    _abi.check(lib.ascan_forward_split_static(cg.data_ptr(), cx.data_ptr(), cout.data_ptr(), rows, T, 3, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(torch.view_as_real(cout), torch.view_as_real(cwant))
    del cg, cx, cout, cwant
    # rows of half a tile, two to a swept tile: the forward kernel needs the ticket only, whatever the number of rows
    rows, T = 40000, 8192
    assert lib.ascan_workspace_bytes(rows, T, 0) > 4 * 1024 * 1024
    hg, hx = torch.rand(rows, T, device=DEVICE), torch.rand(rows, T, device=DEVICE)
    hout, hwant = torch.empty_like(hx), torch.empty_like(hx)
    table = torch.empty(lib.ascan_workspace_bytes(rows, T, 0), dtype=torch.uint8, device=DEVICE)
    _abi.check(lib.ascan_forward_split(hg.data_ptr(), hx.data_ptr(), hwant.data_ptr(), rows, T, 0, 0, table.data_ptr(),
                                       table.numel(), stream))
    _abi.check(lib.ascan_forward_split_static(hg.data_ptr(), hx.data_ptr(), hout.data_ptr(), rows, T, 0, 0, stream))
    torch.cuda.synchronize()
    assert torch.equal(hout, hwant)
    count = ctypes.c_uint(7)
    _abi.check(lib.ascan_static_workspace_timeouts(ctypes.byref(count), stream))
    assert count.value == 0
    del hg, hx, hout, hwant, table
    # validation is that of the other entry points
    assert lib.ascan_forward_split_static(None, x.data_ptr(), out.data_ptr(), 4, 256, 0, 0, stream) == 1
    assert lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), out.data_ptr(), 4, 256, 9, 0, stream) == 3
    assert lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), g.data_ptr(), 4, 256, 0, 0, stream) == 7


def test_static_table_under_graph_capture():
    """After one eager call (which looks the array's address up), the entry point is
    captured into a HIP graph and replayed on new inputs; every replay must equal
    ascan_forward_split on the same inputs."""
    from accelerated_scan import _abi

    lib = _abi.load()
    rows, T = 3, 300000
    nbytes = lib.ascan_workspace_bytes(rows, T, 0)
    assert 0 < nbytes <= 4 * 1024 * 1024
    gen = torch.Generator().manual_seed(7)
    g = torch.empty(rows, T, device=DEVICE)
    x = torch.empty(rows, T, device=DEVICE)
    got, want = torch.empty_like(g), torch.empty_like(g)
    workspace = torch.empty(nbytes, dtype=torch.uint8, device=DEVICE)

    def refill():
        g.copy_(0.9 + 0.1 * torch.rand(rows, T, generator=gen))
        x.copy_(torch.randn(rows, T, generator=gen))

    def run_static():
        stream = torch.cuda.current_stream().cuda_stream
        _abi.check(lib.ascan_forward_split_static(g.data_ptr(), x.data_ptr(), got.data_ptr(), rows, T, 0, 0, stream))

    refill()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run_static()  # outside capture: the first use on this GPU
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        run_static()
    for _ in range(3):
        refill()
        got.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        _abi.check(lib.ascan_forward_split(g.data_ptr(), x.data_ptr(), want.data_ptr(), rows, T, 0, 0,
                                           workspace.data_ptr(), nbytes, torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert torch.equal(got, want)
        ran_out = ctypes.c_uint(99)
        _abi.check(lib.ascan_static_workspace_timeouts(ctypes.byref(ran_out), None))
        assert ran_out.value == 0
