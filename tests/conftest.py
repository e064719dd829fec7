import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT, ROOT / "accelerated-scan_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a HIP device (run on the MI355X box)")


def pytest_sessionstart(session):
    """The libraries are built beforehand (``__graft_entry__.build()``); only when
    none is there at all are they built here, so that a fresh checkout can run."""
    import subprocess

    if not (ROOT / "accelerated-scan_amd" / "accelerated_scan" / "libascan.so").exists():
        subprocess.run(["make", "-j8", "-C", str(ROOT / "accelerated-scan_amd")], check=True, capture_output=True)
    if not (ROOT / "oracle" / "_build" / "libseqscan.so").exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    path = Path(__file__).resolve().parent / "golden" / "ref_scan_golden.npz"
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}
