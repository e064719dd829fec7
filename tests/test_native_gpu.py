"""The C ABI driven from a plain HIP host program (no Python, no torch in the
process): tests/native/abi_check.cpp links libascan.so through include/ascan.h,
allocates with hipMalloc, runs every entry point on its own stream and checks the
results against the sequential fp64 loops of oracle/seqscan.c.

The program is built beforehand (``make -C tests/native`` or
``__graft_entry__.build()``); this test runs it, and builds it first only when
no binary is there.
"""

import subprocess
from pathlib import Path

import pytest

pytestmark = pytest.mark.gpu

BINARY = Path(__file__).resolve().parent / "native" / "abi_check"


def test_c_abi_from_a_plain_hip_program():
    if not BINARY.exists():  # normally built beforehand; build only if nothing is there
        subprocess.run(["make", "-C", str(BINARY.parent)], check=True, capture_output=True, timeout=300)
    run = subprocess.run([str(BINARY)], capture_output=True, text=True, timeout=100)
    assert run.returncode == 0, f"stdout:\n{run.stdout}\nstderr:\n{run.stderr}"
    assert run.stdout.strip().endswith("ok")
