"""Compiles the native libraries in-tree (hipcc for gfx950, g++ for the host layer and for the
Python extension module)."""
import os
import subprocess
import sysconfig

_HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(_HERE, "csrc")
LIBDIR = os.path.join(_HERE, "lib")
EXTENSION = os.path.join(_HERE, "engine_c" + (sysconfig.get_config_var("EXT_SUFFIX") or ".so"))


def build_native(jobs: int = 8, force: bool = False) -> None:
    """Runs ``make`` in ``pccl_amd/csrc``; ``force`` rebuilds every object."""
    if force:
        subprocess.run(["make", "-C", CSRC, "clean"], check=True, stdout=subprocess.DEVNULL)
    subprocess.run(["make", "-C", CSRC, "-j%d" % jobs, "all"], check=True)
    for name in ("libpccl_hip.so", "libpccl_engine.so"):
        path = os.path.join(LIBDIR, name)
        if not os.path.exists(path):
            raise RuntimeError("build did not produce %s" % path)


def build_extension() -> None:
    """``pccl_amd.engine_c``: pybind11 module over ``libpccl_engine.so`` whose ``exeOp`` takes torch
    tensors (the reference builds its ``pccl.engine_c`` the same way, ``setup.py:105-112``).  Host code
    only; links torch's libraries and finds ``libpccl_engine.so`` next to itself at run time."""
    import torch
    from torch.utils import cpp_extension
    root = os.path.dirname(_HERE)
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-fvisibility=hidden", "-D__HIP_PLATFORM_AMD__", "-DUSE_ROCM",
           "-D_GLIBCXX_USE_CXX11_ABI=%d" % int(torch._C._GLIBCXX_USE_CXX11_ABI),
           "-DTORCH_EXTENSION_NAME=engine_c", "-Wno-attributes",
           "-I", os.path.join(CSRC, "host"), "-I", os.path.join(root, "include"), "-I/opt/rocm/include",
           "-I", sysconfig.get_paths()["include"]]
    for inc in cpp_extension.include_paths():
        cmd += ["-isystem", inc]
    cmd += [os.path.join(CSRC, "python", "python_api.cc"), "-o", EXTENSION,
            "-L", LIBDIR, "-lpccl_engine", "-L", torch_lib, "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch", "-ltorch_python",
            "-Wl,-rpath,$ORIGIN/lib", "-Wl,-rpath," + torch_lib]
    subprocess.run(cmd, check=True)
    if not os.path.exists(EXTENSION):
        raise RuntimeError("build did not produce %s" % EXTENSION)
