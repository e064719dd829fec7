"""Wheel build: compiles the gfx950 library with hipcc (the Makefile next to this
file) and ships it, with the C header, inside the ``accelerated_scan`` package.

    python -m pip wheel --no-build-isolation --no-deps -w dist ./accelerated-scan_amd

The wheel carries prebuilt machine code for one GPU architecture, so it is
tagged for the platform it was built on; the reference's wheel is pure Python
and compiles its CUDA source on first import (accelerated_scan/warp.py:13-28).
"""

import shutil
import subprocess
from pathlib import Path

from setuptools import setup
from setuptools.command.build_py import build_py
from wheel.bdist_wheel import bdist_wheel

HERE = Path(__file__).resolve().parent


class BuildWithLibrary(build_py):
    def run(self):
        subprocess.run(["make", "-j8", "-C", str(HERE)], check=True)
        header_dir = HERE / "accelerated_scan" / "include"
        header_dir.mkdir(exist_ok=True)
        shutil.copy2(HERE.parent / "include" / "ascan.h", header_dir / "ascan.h")
        try:
            super().run()
        finally:
            shutil.rmtree(header_dir, ignore_errors=True)


class PlatformWheel(bdist_wheel):
    """The shared library is called through ctypes: any Python 3, this platform only."""

    def finalize_options(self):
        super().finalize_options()
        self.root_is_pure = False

    def get_tag(self):
        return "py3", "none", super().get_tag()[2]


def version():
    for line in (HERE / "accelerated_scan" / "__init__.py").read_text().splitlines():
        if line.startswith("__version__"):
            return line.split('"')[1]
    raise RuntimeError("no __version__ in accelerated_scan/__init__.py")


# Metadata mirrors the reference's pyproject.toml:5-21 (same distribution and
# package names, so that `import accelerated_scan` resolves to this build).
setup(
    name="accelerated-scan",
    version=version(),
    description="First-order associative scan for AMD MI355X (gfx950); drop-in for the accelerated_scan package",
    packages=["accelerated_scan"],
    package_data={"accelerated_scan": ["libascan.so", "include/ascan.h"]},
    install_requires=["torch>=2.9.0"],
    python_requires=">=3.10",
    classifiers=[
        "Programming Language :: Python :: 3",
        "License :: OSI Approved :: MIT License",
        "Operating System :: POSIX :: Linux",
    ],
    cmdclass={"build_py": BuildWithLibrary, "bdist_wheel": PlatformWheel},
)
