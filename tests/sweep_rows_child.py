"""Run by tests/test_scan_gpu.py::test_rows_sharing_swept_tiles_small_shapes in a child
process with ASCAN_SWEEP_ROWS=1 (read once per process): the library then puts 2, 4, 8 or 16
whole rows into every swept tile whenever rows divide a tile, whatever the size of the
tensors, so the hand-over between the waves of each row, tiles whose last rows are missing
and rows with initial states are checked at sizes the fp64 loops finish in seconds."""

import struct
import sys
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
sys.path[:0] = [str(ROOT), str(ROOT / "accelerated-scan_amd")]

import numpy as np  # noqa: E402
import torch  # noqa: E402

from accelerated_scan import _abi  # noqa: E402
from oracle import seqscan  # noqa: E402

DEVICE = "cuda"
ULP = {torch.float32: 1e-5, torch.bfloat16: 2.0**-7, torch.float16: 2.0**-10}
PER_WAVE = {torch.float32: 1024, torch.bfloat16: 2048, torch.float16: 2048}  # elements (4 KiB)


def np32(t):
    return t.float().cpu().numpy()


def close(name, got, want, dtype):
    scale = max(1.0, float(np.abs(want).max()))
    np.testing.assert_allclose(np32(got), want, rtol=ULP[dtype], atol=ULP[dtype] * scale, err_msg=name)


def tickets_drawn(table):
    """The ticket counter sits behind the 64-byte header."""
    return struct.unpack("<Q", bytes(table[64:72].cpu().tolist()))[0]


def main():
    lib = _abi.load()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    checked = 0
    for dtype in (torch.float32, torch.bfloat16, torch.float16):
        for per_tile in (2, 4, 8, 16):
            for rows in (1, 37, 2 * per_tile):
                T = PER_WAVE[dtype] * (16 // per_tile)
                gen = torch.Generator().manual_seed(1000 * per_tile + rows)
                gates = torch.rand(rows, T, generator=gen).to(dtype)
                tokens = torch.randn(rows, T, generator=gen).to(dtype)
                grad_out = torch.randn(rows, T, generator=gen).to(dtype)
                start = torch.randn(rows, generator=gen).to(dtype)
                g, x, d, s = (t.to(DEVICE) for t in (gates, tokens, grad_out, start))
                what = f"{dtype} rows={rows} T={T} ({per_tile} rows per tile)"
                units = (rows + per_tile - 1) // per_tile
                for reverse in (False, True):
                    out, dg, dx = (torch.empty_like(g) for _ in range(3))
                    ds = torch.empty_like(s)
                    tables = [torch.ones(4096, dtype=torch.uint8, device=DEVICE) for _ in range(2)]  # garbage
                    _abi.forward(g, x, out, reverse, workspace=tables[0], initial=s)
                    _abi.backward(g, out, d, dg, dx, workspace=tables[1], initial=s, d_initial=ds, reverse=reverse)
                    torch.cuda.synchronize()
                    for table in tables:
                        # every workgroup draws until it is turned away: tiles + workgroups tickets, of
                        # tiles that hold per_tile rows each
                        assert tickets_drawn(table) == units + min(units, cus), (what, tickets_drawn(table), units)
                        assert _abi.workspace_timeouts(table) == 0
                    t_out = seqscan.forward_from(np32(gates), np32(tokens), np32(start), reverse=reverse)
                    close(what + " out", out, t_out, dtype)
                    t_dg, t_dx, t_ds = seqscan.backward_from(np32(gates), np32(out), np32(start), np32(grad_out),
                                                             reverse=reverse)
                    close(what + " d_tokens", dx, t_dx, dtype)
                    close(what + " d_gates", dg, t_dg, dtype)
                    close(what + " d_initial", ds, t_ds, dtype)
                    checked += 1
    # the gates with a non-linearity, fp32: the backward kernels of the two gates with values take 2 KiB per
    # wave, so their rows are half as long per wave
    for gate, fwd, bwd, with_values in (
            (_abi.GATE_SIGMOID, seqscan.forward_sigmoid, seqscan.backward_sigmoid, False),
            (_abi.GATE_EXP, seqscan.forward_exp, seqscan.backward_exp, False),
            (_abi.GATE_SIGMOID_LERP, seqscan.forward_lerp, seqscan.backward_lerp, True),
            (_abi.GATE_EXP_NORM, seqscan.forward_expnorm, seqscan.backward_expnorm, True)):
        for rows, T in ((5, 4096), (9, 1024), (3, 8192)):
            gen = torch.Generator().manual_seed(gate * 100 + rows)
            z = torch.randn(rows, T, generator=gen) + 2.0
            if gate in (_abi.GATE_EXP, _abi.GATE_EXP_NORM):
                z = -torch.rand(rows, T, generator=gen) * 0.2 - 1e-3  # logarithms of gates below one
            tokens = torch.randn(rows, T, generator=gen)
            grad_out = torch.randn(rows, T, generator=gen)
            start = torch.randn(rows, generator=gen)
            zg, x, d, s = (t.to(DEVICE) for t in (z, tokens, grad_out, start))
            out, dz, dx = (torch.empty_like(zg) for _ in range(3))
            ds = torch.empty_like(s)
            tables = [torch.zeros(4096, dtype=torch.uint8, device=DEVICE) for _ in range(2)]
            what = f"gate {gate} rows={rows} T={T}"
            per_wave = (1024, 512 if with_values else 1024)  # forward, backward
            shared = [T // n <= 8 for n in per_wave]  # a row on at most half a tile's waves: rows share tiles
            _abi.forward_gated(zg, x, out, gate, workspace=tables[0], initial=s)
            if with_values:
                _abi.backward_gated_values(zg, x, out, d, dz, dx, gate, workspace=tables[1], initial=s, d_initial=ds)
            else:
                _abi.backward_gated(zg, out, d, dz, dx, gate, workspace=tables[1], initial=s, d_initial=ds)
            torch.cuda.synchronize()
            assert [tickets_drawn(t) > 0 for t in tables] == shared, what
            assert all(_abi.workspace_timeouts(t) == 0 for t in tables), what
            close(what + " out", out, fwd(np32(z), np32(tokens), np32(start)), torch.float32)
            if with_values:
                t_dz, t_dx, t_ds = bwd(np32(z), np32(tokens), np32(out), np32(grad_out), np32(start))
            else:
                t_dz, t_dx, t_ds = bwd(np32(z), np32(out), np32(grad_out), np32(start))
            close(what + " d_gate_inputs", dz, t_dz, torch.float32)
            close(what + " d_tokens", dx, t_dx, torch.float32)
            close(what + " d_initial", ds, t_ds, torch.float32)
            checked += 1
    print("checked", checked)


if __name__ == "__main__":
    main()
