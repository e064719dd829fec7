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

    library = ROOT / "accelerated-scan_amd" / "accelerated_scan" / "libascan.so"
    if not library.exists():
        subprocess.run(["make", "-j8", "-C", str(ROOT / "accelerated-scan_amd")], check=True, capture_output=True)
    else:
        # a library older than its sources is tested as it is, but not silently
        sources = list((ROOT / "accelerated-scan_amd" / "csrc").glob("*")) + [ROOT / "include" / "ascan.h"]
        newer = [p.name for p in sources if p.stat().st_mtime > library.stat().st_mtime]
        if newer:
            import warnings

            warnings.warn(f"libascan.so is older than {', '.join(sorted(newer))}: run `make -C accelerated-scan_amd` "
                          "(or __graft_entry__.build()) to test the current sources")
    if not (ROOT / "oracle" / "_build" / "libseqscan.so").exists():
        subprocess.run(["make", "-C", str(ROOT / "oracle")], check=True, capture_output=True)


@pytest.fixture(scope="session")
def golden():
    import numpy as np

    path = Path(__file__).resolve().parent / "golden" / "ref_scan_golden.npz"
    with np.load(path, allow_pickle=False) as z:
        return {k: z[k] for k in z.files}
