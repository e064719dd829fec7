"""The wheel, exercised and not only listed: built, unpacked into a directory of
its own, and imported by a child process that has only that directory (and the
oracle) on its path -- the package the reference ships as `accelerated-scan`
(pyproject.toml:1-24 of the reference).  The child compares warp.scan,
gated.sigmoid_scan and ref.scan with the oracle on the GPU."""

import subprocess
import sys
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

ROOT = Path(__file__).resolve().parents[1]

CHILD = r"""
import sys
site, root = sys.argv[1], sys.argv[2]
sys.path[:0] = [site, root]            # the unpacked wheel first; the repository root only for oracle/
import numpy as np
import torch
import accelerated_scan
from accelerated_scan import _abi
from accelerated_scan.warp import scan
from accelerated_scan.gated import sigmoid_scan
from accelerated_scan.ref import scan as ref_scan_name
from oracle import seqscan

assert accelerated_scan.__file__.startswith(site), accelerated_scan.__file__
assert str(_abi.library_path()).startswith(site), _abi.library_path()
gen = torch.Generator().manual_seed(11)
for shape in ((2, 5, 3000), (1, 3, 70001)):
    gates = torch.rand(shape, generator=gen)
    tokens = torch.randn(shape, generator=gen)
    grad = torch.randn(shape, generator=gen)
    rows, T = shape[0] * shape[1], shape[2]
    want = seqscan.forward(gates.reshape(rows, T).numpy(), tokens.reshape(rows, T).numpy()).reshape(shape)
    dg_want, dx_want = seqscan.backward(gates.reshape(rows, T).numpy(), want.reshape(rows, T), grad.reshape(rows, T).numpy())
    g = gates.cuda().requires_grad_()
    x = tokens.cuda().requires_grad_()
    out = scan(g, x)
    out.backward(grad.cuda())
    scale = float(np.abs(want).max())
    np.testing.assert_allclose(out.detach().cpu().numpy(), want, rtol=2e-5, atol=2e-5 * scale)
    np.testing.assert_allclose(x.grad.cpu().numpy(), dx_want.reshape(shape), rtol=2e-5, atol=2e-5 * float(np.abs(dx_want).max()))
    np.testing.assert_allclose(g.grad.cpu().numpy(), dg_want.reshape(shape), rtol=2e-5, atol=2e-5 * float(np.abs(dg_want).max()))
    again = ref_scan_name(gates.cuda(), tokens.cuda())
    np.testing.assert_allclose(again.cpu().numpy(), want, rtol=2e-5, atol=2e-5 * scale)
    logits = torch.logit(gates.clamp(1e-4, 1 - 1e-4))
    fused = sigmoid_scan(logits.cuda(), tokens.cuda())
    want_sig = seqscan.forward(torch.sigmoid(logits.double()).float().reshape(rows, T).numpy(), tokens.reshape(rows, T).numpy())
    np.testing.assert_allclose(fused.cpu().numpy().reshape(rows, T), want_sig, rtol=2e-5, atol=2e-5 * float(np.abs(want_sig).max()))
print("wheel ok")
"""


def test_installed_wheel_runs_the_scans(tmp_path):
    src = ROOT / "accelerated-scan_amd"
    subprocess.run(
        [sys.executable, "setup.py", "-q", "egg_info", "--egg-base", str(tmp_path),
         "bdist_wheel", "-d", str(tmp_path / "dist"), "-b", str(tmp_path / "build")],
        cwd=src, check=True, capture_output=True,
    )
    (wheel,) = (tmp_path / "dist").glob("*.whl")
    site = tmp_path / "site"
    subprocess.run([sys.executable, "-m", "pip", "install", "-q", "--no-index", "--no-deps", "--no-cache-dir",
                    "--target", str(site), str(wheel)], check=True, capture_output=True)
    assert (site / "accelerated_scan" / "libascan.so").exists()
    done = subprocess.run([sys.executable, "-c", CHILD, str(site), str(ROOT)], capture_output=True, text=True,
                          timeout=110, cwd=tmp_path)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "wheel ok" in done.stdout
