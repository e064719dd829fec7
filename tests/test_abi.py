"""CPU tests of the drop-in boundary: the shared library loads, exports every
symbol include/ascan.h declares, rejects bad arguments by return code before
touching the GPU, and the Python operators validate like the reference's
(accelerated_scan/warp.py:41-44, warp.cuh:394-421, complex.py:160-161).
No kernel is launched here.
"""

import ctypes
import re
from pathlib import Path

import pytest
import torch

from accelerated_scan import _abi

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "ascan.h"


def declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(ascan_[a-z0-9_]+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(str(_abi.library_path()))
    names = declared_functions()
    assert set(names) >= {"ascan_forward", "ascan_backward", "ascan_status_string", "ascan_abi_version"}
    for name in names:
        assert hasattr(lib, name), name
    assert set(_abi.exported_symbols()) == set(names)


def test_abi_version_and_status_strings():
    lib = _abi.load()
    assert lib.ascan_abi_version() == _abi.ABI_VERSION
    texts = {lib.ascan_status_string(i).decode() for i in range(9)}
    assert len(texts) == 9 and "ok" in texts
    assert lib.ascan_status_string(99).decode() == "unknown status"


def test_argument_validation_returns_codes():
    lib = _abi.load()
    buf = ctypes.create_string_buffer(64)
    p = ctypes.addressof(buf)
    # unknown dtype
    assert lib.ascan_forward(p, p, p, 1, 4, 7, 0, None) == 3
    assert lib.ascan_backward(p, p, p, p, p, 1, 4, -1, None) == 3
    # unknown gate activation, or one the dtype does not have
    assert lib.ascan_forward_gated(p, p, None, p, 1, 4, 0, 5, None, 0, None) == 6
    assert lib.ascan_forward_gated(p, p, None, p, 1, 4, 3, 1, None, 0, None) == 6
    assert lib.ascan_backward_gated(p, p, None, p, p, p, None, 1, 4, 4, 1, None, 0, None) == 6
    # negative sizes, too many rows
    assert lib.ascan_forward(p, p, p, -1, 4, 0, 0, None) == 2
    assert lib.ascan_forward(p, p, p, 1, -4, 0, 0, None) == 2
    assert lib.ascan_forward(p, p, p, 2**31, 4, 0, 0, None) == 2
    assert lib.ascan_forward(p, p, p, 2**31 - 1, 2**40, 0, 0, None) == 2  # rows * seqlen beyond the address space
    assert lib.ascan_forward(p, p, p, 1, 2**63 - 1, 0, 0, None) == 2
    assert lib.ascan_workspace_bytes(1, 2**63 - 1, 0) == 0
    assert lib.ascan_backward(p, p, p, p, p, 1, -1, 0, None) == 2
    # empty problems succeed without looking at the pointers
    assert lib.ascan_forward(None, None, None, 0, 4, 0, 0, None) == 0
    assert lib.ascan_forward(None, None, None, 4, 0, 0, 0, None) == 0
    assert lib.ascan_backward(None, None, None, None, None, 0, 0, 3, None) == 0
    # null pointers
    assert lib.ascan_forward(None, p, p, 1, 4, 0, 0, None) == 1
    assert lib.ascan_forward(p, p, None, 1, 4, 0, 0, None) == 1
    assert lib.ascan_backward(p, p, p, p, None, 1, 4, 0, None) == 1
    # element misalignment
    assert lib.ascan_forward(p + 2, p, p, 1, 4, 0, 0, None) == 4
    assert lib.ascan_forward(p + 1, p, p, 1, 4, 1, 0, None) == 4
    assert lib.ascan_forward(p + 4, p, p, 1, 4, 3, 0, None) == 4
    assert lib.ascan_backward(p, p, p, p + 2, p, 1, 4, 0, None) == 4
    # the reverse scan's backward pass validates like the forward-time one
    assert lib.ascan_backward_reverse(p, p, None, p, p, p, None, -1, 4, 0, None, 0, None) == 2
    assert lib.ascan_backward_reverse(None, None, None, None, None, None, None, 0, 4, 0, None, 0, None) == 0
    assert lib.ascan_backward_reverse(p, p, None, p, None, p, None, 1, 4, 0, None, 0, None) == 1
    assert lib.ascan_backward_reverse(p, p, None, p, p + 2, p, None, 1, 4, 0, None, 0, None) == 4
    assert lib.ascan_backward_reverse(p, p, None, p, p, p, None, 1, 4, 9, None, 0, None) == 3


def test_overlapping_buffers_are_refused():
    """An output that overlaps an input or another output is refused by a host-side
    interval check before anything is launched (include/ascan.h: ASCAN_ERR_OVERLAP)."""
    lib = _abi.load()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    p += -p % 64
    n = 16  # one row of 16 fp32 elements = 64 bytes
    assert lib.ascan_forward(p, p + 64, p, 1, n, 0, 0, None) == 7              # out is gates
    assert lib.ascan_forward(p, p + 64, p + 64 + 60, 1, n, 0, 0, None) == 7    # out starts inside tokens
    assert lib.ascan_forward(p + 60, p + 256, p, 1, n, 0, 0, None) == 7        # gates start inside out
    assert lib.ascan_forward_from(p, p + 64, p + 128 + 32, p + 128, 1, n, 0, 0, None, 0, None) == 7  # initial inside out
    assert lib.ascan_backward(p, p + 64, p + 128, p + 128, p + 256, 1, n, 0, None) == 7      # d_gates is grad_out
    assert lib.ascan_backward(p, p + 64, p + 128, p + 256, p + 256 + 32, 1, n, 0, None) == 7  # the two outputs overlap
    assert lib.ascan_backward_from(p, p + 64, None, p + 128, p + 192, p + 256, p + 192 + 8, 1, n, 0, None, 0, None) == 7
    assert lib.ascan_backward_reverse(p, p + 64, None, p + 128, p + 192, p + 256, p + 192 + 8, 1, n, 0, None, 0, None) == 7
    # complex gates with real tokens: the token buffers are half as long
    assert lib.ascan_forward(p, p + 256, p + 256 + 56, 1, n, 4, 0, None) == 7   # 16 c64 = 128 bytes, tokens 64 bytes
    # bf16: 32 bytes per row; ranges that only touch are fine for the check (the
    # call then stops at the next one, here the missing d_tokens)
    assert lib.ascan_backward(p, p + 32, p + 64, p + 96, None, 1, n, 1, None) == 1


def test_workspace_sizing_and_split_entry_validation():
    lib = _abi.load()
    buf = ctypes.create_string_buffer(256)
    p = ctypes.addressof(buf)
    # short rows, and a complex row per compute unit: the plain kernels are the right choice
    assert lib.ascan_workspace_bytes(12288, 4096, 0) == 0
    assert lib.ascan_workspace_bytes(4096, 16384, 1) == 0
    assert lib.ascan_workspace_bytes(12288, 12288, 1) == 0
    assert lib.ascan_workspace_bytes(4, 4096, 0) == 0
    assert lib.ascan_workspace_bytes(256, 65536, 3) == 0
    # long rows in a real dtype are swept in memory order, however many there are (fp32 from 32 KiB on:
    # the backward kernel gains from half-full 64 KiB tiles; 16-bit from 64 KiB on)
    assert lib.ascan_workspace_bytes(12288, 65536, 0) == 128 + 12288 * (65536 // 8192 + 1) * 64
    assert lib.ascan_workspace_bytes(12288, 8192, 0) > 0
    assert lib.ascan_workspace_bytes(12288, 32768, 1) > 0
    # many complex rows of 64 KiB and more: the backward kernel is swept, and the forward kernel from two tiles on
    assert lib.ascan_workspace_bytes(6144, 65536, 3) == 128 + 6144 * (65536 // 4096 + 1) * 64
    assert lib.ascan_workspace_bytes(6144, 262144, 3) == 128 + 6144 * (262144 // 4096 + 1) * 64
    assert lib.ascan_workspace_bytes(4096, 8192, 4) > 0
    # 16-bit rows of exactly half a tile, two to a swept tile, once the tensors reach 256 MiB
    assert lib.ascan_workspace_bytes(12288, 16384, 1) > 0
    assert lib.ascan_workspace_bytes(12288, 16384, 2) > 0
    assert lib.ascan_workspace_bytes(4, 1 << 20, 9) == 0  # unknown dtype
    assert lib.ascan_workspace_bytes(-1, 1 << 20, 0) == 0
    # few long rows: header (64 bytes) + the ticket line (64 bytes)
    # + one 64-byte record per (row, smallest tile)
    nbytes = lib.ascan_workspace_bytes(4, 1 << 20, 0)
    assert nbytes == 64 + 64 + 4 * ((1 << 20) // 8192 + 1) * 64
    assert lib.ascan_workspace_bytes(4, 1 << 20, 3) > 0  # complex rows too, when they are few
    assert lib.ascan_workspace_bytes(4, 1 << 20, 1) < nbytes  # 16-bit tiles hold more elements
    # the split entry points validate like the plain ones, before touching the GPU
    assert lib.ascan_forward_split(p, p, p, 1, 4, 7, 0, None, 0, None) == 3
    assert lib.ascan_forward_split(None, p, p, 1, 4, 0, 0, None, 0, None) == 1
    assert lib.ascan_forward_split(p, p, p, -1, 4, 0, 0, None, 0, None) == 2
    assert lib.ascan_forward_split(None, None, None, 0, 4, 0, 0, None, 0, None) == 0
    assert lib.ascan_backward_split(p, p, p, p, p + 2, 1, 4, 0, None, 0, None) == 4
    assert lib.ascan_backward_split(p, p, p, p, None, 1, 4, 0, None, 0, None) == 1
    # the header accessor reads the count of waits that ran out from a host copy
    header = (ctypes.c_uint32 * 16)()
    header[4] = 3
    assert lib.ascan_workspace_timeouts(ctypes.addressof(header)) == 3


def test_static_workspace_entry_point_validates_before_touching_the_gpu():
    """ascan_forward_split_static refuses problems whose table exceeds the static
    array, and validates like the other entry points, without a GPU."""
    lib = _abi.load()
    buf = ctypes.create_string_buffer(4096)
    p = ctypes.addressof(buf)
    limit = 4 * 1024 * 1024  # ASCAN_STATIC_WORKSPACE_BYTES
    assert lib.ascan_workspace_bytes(128, 1 << 24, 0) > limit
    assert lib.ascan_forward_split_static(p, p + 1024, p + 2048, 128, 1 << 24, 0, 0, None) == 8
    assert 0 < lib.ascan_workspace_bytes(64, 1 << 22, 0) <= limit
    assert lib.ascan_forward_split_static(None, p + 1024, p + 2048, 64, 1 << 22, 0, 0, None) == 1
    assert lib.ascan_forward_split_static(p, p + 1024, p + 2048, 3, 1 << 20, 9, 0, None) == 3
    assert lib.ascan_forward_split_static(p, p + 1024, p + 2048, -3, 1 << 20, 0, 0, None) == 2
    assert lib.ascan_forward_split_static(None, None, None, 0, 1 << 20, 0, 0, None) == 0
    assert "static workspace" in lib.ascan_status_string(8).decode()


def test_status_becomes_runtime_error():
    with pytest.raises(RuntimeError, match="unsupported dtype"):
        _abi.check(3)
    _abi.check(0)
    with pytest.raises(RuntimeError, match="unsupported tensor dtype"):
        _abi.dtype_code(torch.float64)


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setenv("ASCAN_LIBRARY", str(tmp_path / "nope.so"))
    monkeypatch.setattr(_abi, "_lib", None)
    with pytest.raises(ImportError, match="HIP library not found"):
        _abi.load()


def test_warp_rejects_host_tensors_and_bad_shapes():
    from accelerated_scan import warp

    g = torch.rand(1, 2, 8)
    x = torch.rand(1, 2, 8)
    with pytest.raises(RuntimeError, match="device tensor"):
        warp.scan(g, x)
    with pytest.raises(RuntimeError, match="device tensor"):
        warp.warpscan_backward(g, g, g, g, g)
    with pytest.raises(AssertionError):
        warp.scan(g, torch.rand(1, 2, 9))
    with pytest.raises(AssertionError):
        warp.scan(torch.rand(2, 1, 8, 2)[..., 0], x.reshape(2, 1, 8))
    with pytest.raises(AssertionError):
        warp.scan(g, torch.rand(1, 2, 16)[:, :, ::2])


def test_scalar_and_complex_validation():
    from accelerated_scan import complex as cscan
    from accelerated_scan import scalar

    g = torch.rand(1, 2, 8)
    with pytest.raises(RuntimeError, match="device tensor"):
        scalar.scan(g, g)
    with pytest.raises(TypeError, match="forget must be a complex tensor"):
        cscan.scan(g, g)
    gc = torch.polar(torch.rand(1, 2, 8), torch.rand(1, 2, 8))
    with pytest.raises(RuntimeError, match="device tensor"):
        cscan.scan(gc, g)
    with pytest.raises(AssertionError):
        cscan.scan(gc, torch.rand(1, 2, 9))


def test_module_surface_matches_reference():
    import accelerated_scan
    from accelerated_scan import complex as cscan
    from accelerated_scan import scalar, warp

    assert accelerated_scan.__version__ == "0.3.1"
    for name in ("scan", "Scan", "scan_forward", "warpscan_forward", "warpscan_backward"):
        assert hasattr(warp, name)
    for mod in (scalar, cscan):
        assert hasattr(mod, "scan") and hasattr(mod, "Scan")
        assert issubclass(mod.Scan, torch.autograd.Function)


def test_wheel_carries_library_and_header(tmp_path):
    """The wheel is a platform wheel with the prebuilt library and the C header
    inside the package, under the reference's distribution name
    (pyproject.toml:6 of the reference)."""
    import subprocess
    import sys
    import zipfile

    src = ROOT / "accelerated-scan_amd"
    subprocess.run(
        [sys.executable, "setup.py", "-q", "egg_info", "--egg-base", str(tmp_path),
         "bdist_wheel", "-d", str(tmp_path / "dist"), "-b", str(tmp_path / "build")],
        cwd=src, check=True, capture_output=True,
    )
    (wheel,) = (tmp_path / "dist").glob("*.whl")
    assert wheel.name.startswith("accelerated_scan-") and wheel.name.endswith("-py3-none-linux_x86_64.whl")
    names = {n.split("accelerated_scan/", 1)[1] for n in zipfile.ZipFile(wheel).namelist() if "accelerated_scan/" in n}
    assert {"libascan.so", "include/ascan.h", "__init__.py", "_abi.py", "_ops.py", "warp.py", "scalar.py",
            "complex.py", "stateful.py", "gated.py", "ref.py"} <= names
    assert not (src / "accelerated_scan" / "include").exists()  # the header copy is temporary
