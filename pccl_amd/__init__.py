"""pccl_amd -- MI355X (gfx950) reduce-copy core behind PCCL's plugin/engine interface.

The product is two native libraries built in-tree under ``pccl_amd/lib``:

* ``libpccl_hip.so``    hand-written HIP kernels + the C ABI of ``include/pccl_hip.h``
* ``libpccl_engine.so`` the C++ host layer (TypeRegistry, DeviceBase plugins, Engine)
  that reaches the GPU only through that C ABI; C ABI in ``include/pccl_engine.h``

This Python package is plumbing: ctypes bindings so tests, the benchmark and Python
callers can reach the C ABI with torch tensors as device memory.  There is no CPU
fallback: loading fails loudly when the native libraries are missing.
"""
from . import hip  # noqa: F401

__all__ = ["hip"]
