"""Build and install the MI355X `bsi_ops` replacement: `pip install .` (or `python setup.py build`).

Counterpart of the reference's `bsi_ops/setup.py:1-55`, which compiles its CUDA sources into one extension module
named `bsi_ops`.  Here the device code is `libbsi_hip.so` (hand-written HIP for gfx950, built by hipcc through
`bsipytorch_amd/csrc/Makefile`, together with `libbsi_reference_launchers.so`, the reference's own `launch_*`
symbols forwarded to it); both are installed inside the `bsipytorch_amd` package, and the top-level module `bsi_ops`
re-exports the reference's API, so `import bsi_ops` works as it does with the reference's extension.
Needs ROCm's hipcc on PATH; `BSI_HIP_ARCH` overrides the target (default gfx950).
"""
import os
import subprocess

from setuptools import setup
from setuptools.command.build_py import build_py

ROOT = os.path.dirname(os.path.abspath(__file__))


class BuildWithHip(build_py):
    """Runs the Makefile first, so that the shared libraries exist when the package data is collected."""

    def run(self):
        jobs = str(min(16, os.cpu_count() or 1))
        cmd = ["make", "-j", jobs, "-C", os.path.join(ROOT, "bsipytorch_amd", "csrc")]
        if os.environ.get("BSI_HIP_ARCH"):
            cmd.append("ARCH=" + os.environ["BSI_HIP_ARCH"])
        subprocess.run(cmd, check=True)
        super().run()


setup(
    name="bsi_ops_mi355x",
    version="0.2.0",
    description="MI355X-native bsi_ops: BSI builder, EWAH codec and the fixed-bit chunk-scale dot behind the reference's API",
    packages=["bsipytorch_amd", "bsipytorch_amd.benchmarks"],
    py_modules=["bsi_ops"],
    package_data={"bsipytorch_amd": ["libbsi_hip.so", "libbsi_reference_launchers.so"]},
    include_package_data=False,
    python_requires=">=3.9",
    install_requires=[],  # torch (ROCm build) supplies device memory and streams; it is not pulled in from here
    cmdclass={"build_py": BuildWithHip},
    zip_safe=False,
)
