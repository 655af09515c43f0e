"""Compiles the native libraries in-tree (hipcc for gfx950, g++ for the host layer)."""
import os
import subprocess

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIBDIR = os.path.join(_HERE, "lib")


def build_native(jobs: int = 8, force: bool = False) -> None:
    """Runs ``make`` in ``pccl_amd/csrc``; ``force`` rebuilds every object."""
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", CSRC, "-j%d" % jobs, "all"], check=True)
    for name in ("libpccl_hip.so", "libpccl_engine.so"):
        path = os.path.join(LIBDIR, name)
        if not os.path.exists(path):
            raise RuntimeError("build did not produce %s" % path)
