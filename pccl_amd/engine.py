"""ctypes binding of ``libpccl_engine.so`` (C ABI in ``include/pccl_engine.h``).

:class:`Engine` offers the methods the reference exports to Python
(``csrc/python_api.cc:13-20``): ``initEngine``, ``regOp``, ``exeOp``, ``exportEndpoint``,
``joinCluster``, ``exitCluster``; ``exeOp`` takes torch tensors (anything with ``data_ptr()``,
``numel()`` and ``element_size()``).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpccl_engine.so")


class EngineError(RuntimeError):
    pass


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("%s is missing: build it first (there is no fallback)" % LIB_PATH)
        from . import hip
        hip.lib()  # libpccl_hip.so first, with RTLD_GLOBAL
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, cl, cs = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_char_p
        P = ctypes.POINTER
        sigs = {
            "pccl_engine_create": [ci, ci, P(vp)],
            "pccl_engine_destroy": [vp],
            "pccl_engine_init": [vp],
            "pccl_engine_reg_op": [vp, cs, cs],
            "pccl_engine_reg_op_text": [vp, cs, cs],
            "pccl_engine_exe_op": [vp, cs, vp, cl, vp, cl, vp],
            "pccl_engine_wait_op": [vp, cs, vp],
            "pccl_engine_get_dev_buffer": [vp, cs, P(vp), P(vp), P(cl)],
            "pccl_engine_op_info": [vp, cs, P(ci), P(ci), P(cl), P(ci)],
            "pccl_engine_export_endpoint": [vp, cs, ci],
            "pccl_engine_join_cluster": [vp, cs],
            "pccl_engine_exit_cluster": [vp],
            "pccl_engine_reduce_copy": [cs, cs, P(vp), ci, P(vp), ci, cl, vp],
            "pccl_registry_type_id": [cs, P(ci)],
            "pccl_registry_type_name": [ci, cs, ci],
            "pccl_registry_register": [ci, cs, P(ci)],
            "pccl_registry_register_compat": [cs, cs],
            "pccl_registry_is_compatible": [cs, cs, P(ci)],
            "pccl_registry_device_types": [cs, ci],
            "pccl_device_allocator_available": [cs, P(ci)],
            "pccl_device_allocate": [cs, cl, P(vp)],
            "pccl_device_deallocate": [cs, vp],
            "pccl_device_ipc_available": [cs, P(ci)],
            "pccl_env_list_opt": [cs, ci],
            "pccl_env_get": [cs, cs, ci],
            "pccl_env_register_opt": [cs],
            "pccl_schedule_write_ring_allreduce": [cs, cs, cs, ci, cl],
            "pccl_schedule_write_direct_allreduce": [cs, cs, cs, ci, cl],
            "pccl_schedule_write_collective": [cs, cs, cs, cs, ci, cl, ci],
            "pccl_schedule_write_small_message": [cs, cs, ci, ci, ci, ctypes.c_ulong, cl, cl],
            "pccl_schedule_inspect": [cs, P(ci), P(ci), P(cl), P(ci), ci],
        }
        for name, args in sigs.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = ci
        L.pccl_engine_last_error.restype = cs
        L.pccl_engine_last_error.argtypes = []
        _lib = L
    return _lib


def _check(rc):
    if rc != 0:
        raise EngineError(lib().pccl_engine_last_error().decode())


def _b(s):
    return s.encode() if isinstance(s, str) else s


def _addr(x):
    if x is None:
        return None
    return int(x.data_ptr()) if hasattr(x, "data_ptr") else int(x)


class Engine:
    def __init__(self, rank, world_size):
        self._h = ctypes.c_void_p(None)
        _check(lib().pccl_engine_create(rank, world_size, ctypes.byref(self._h)))

    def initEngine(self):
        _check(lib().pccl_engine_init(self._h))

    def regOp(self, name, filepath):
        _check(lib().pccl_engine_reg_op(self._h, _b(name), _b(filepath)))

    def regOpText(self, name, text):
        _check(lib().pccl_engine_reg_op_text(self._h, _b(name), _b(text)))

    def exeOp(self, name, input, output, stream=None):
        nin = input.numel() * input.element_size()
        nout = output.numel() * output.element_size()
        _check(lib().pccl_engine_exe_op(self._h, _b(name), ctypes.c_void_p(_addr(input)), nin,
                                        ctypes.c_void_p(_addr(output)), nout, ctypes.c_void_p(_addr(stream))))

    def waitOp(self, name, stream=None):
        _check(lib().pccl_engine_wait_op(self._h, _b(name), ctypes.c_void_p(_addr(stream))))

    def opInfo(self, name):
        n, d, e, b = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_long(0), ctypes.c_int(0)
        _check(lib().pccl_engine_op_info(self._h, _b(name), ctypes.byref(n), ctypes.byref(d), ctypes.byref(e), ctypes.byref(b)))
        return {"n_ops": n.value, "devices": d.value, "elems_per_device": e.value, "elem_bytes": b.value}

    def getDevBuffer(self, device_name):
        ws, sig, nb = ctypes.c_void_p(None), ctypes.c_void_p(None), ctypes.c_long(0)
        _check(lib().pccl_engine_get_dev_buffer(self._h, _b(device_name), ctypes.byref(ws), ctypes.byref(sig), ctypes.byref(nb)))
        return ws.value, sig.value, nb.value

    def exportEndpoint(self):
        buf = ctypes.create_string_buffer(4096)
        _check(lib().pccl_engine_export_endpoint(self._h, buf, 4096))
        return buf.value.decode()

    def joinCluster(self, master_endpoint):
        _check(lib().pccl_engine_join_cluster(self._h, _b(master_endpoint)))

    def exitCluster(self):
        _check(lib().pccl_engine_exit_cluster(self._h))

    def close(self):
        if self._h:
            _check(lib().pccl_engine_destroy(self._h))
            self._h = ctypes.c_void_p(None)

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def reduce_copy(dtype, compute, ins, outs, count, stream=None):
    """One reduce-copy through the plugin layer (registry names -> HipExecutor -> C ABI)."""
    a_in = (ctypes.c_void_p * max(len(ins), 1))(*[_addr(x) for x in ins])
    a_out = (ctypes.c_void_p * max(len(outs), 1))(*[_addr(x) for x in outs])
    _check(lib().pccl_engine_reduce_copy(_b(dtype), _b(compute), a_in, len(ins), a_out, len(outs), count,
                                         ctypes.c_void_p(_addr(stream))))


# ---- registry / plugins / options ------------------------------------------------------------

KINDS = {"primitive": 0, "data": 1, "compute": 2, "device": 3, "executor": 4}


def type_id(name):
    v = ctypes.c_int(0)
    _check(lib().pccl_registry_type_id(_b(name), ctypes.byref(v)))
    return v.value


def type_name(type_id_):
    buf = ctypes.create_string_buffer(256)
    _check(lib().pccl_registry_type_name(type_id_, buf, 256))
    return buf.value.decode()


def register_type(kind, name):
    v = ctypes.c_int(0)
    _check(lib().pccl_registry_register(KINDS[kind], _b(name), ctypes.byref(v)))
    return v.value


def register_compatibility(executor, name):
    _check(lib().pccl_registry_register_compat(_b(executor), _b(name)))


def is_compatible(executor, name):
    v = ctypes.c_int(0)
    _check(lib().pccl_registry_is_compatible(_b(executor), _b(name), ctypes.byref(v)))
    return bool(v.value)


def device_types():
    buf = ctypes.create_string_buffer(4096)
    _check(lib().pccl_registry_device_types(buf, 4096))
    return [x for x in buf.value.decode().split("\n") if x]


def allocator_available(device):
    v = ctypes.c_int(0)
    _check(lib().pccl_device_allocator_available(_b(device), ctypes.byref(v)))
    return bool(v.value)


def ipc_available(device):
    v = ctypes.c_int(0)
    _check(lib().pccl_device_ipc_available(_b(device), ctypes.byref(v)))
    return bool(v.value)


def allocate(device, nbytes):
    p = ctypes.c_void_p(None)
    _check(lib().pccl_device_allocate(_b(device), nbytes, ctypes.byref(p)))
    return p.value


def deallocate(device, ptr):
    _check(lib().pccl_device_deallocate(_b(device), ctypes.c_void_p(ptr)))


class LaunchEnvironments:
    """utils.LaunchEnvironments of csrc/python_api.cc:24-27."""

    @staticmethod
    def listOpt():
        buf = ctypes.create_string_buffer(4096)
        _check(lib().pccl_env_list_opt(buf, 4096))
        return [x for x in buf.value.decode().split("\n") if x]

    @staticmethod
    def registerOpt(name):
        _check(lib().pccl_env_register_opt(_b(name)))

    @staticmethod
    def getEnv(name):
        buf = ctypes.create_string_buffer(65536)
        _check(lib().pccl_env_get(_b(name), buf, 65536))
        return buf.value.decode()


# ---- native schedule generators ---------------------------------------------------------------

def write_ring_allreduce(path, dtype, compute, devices, chunk_elems):
    _check(lib().pccl_schedule_write_ring_allreduce(_b(path), _b(dtype), _b(compute), devices, chunk_elems))


def write_direct_allreduce(path, dtype, compute, devices, slice_elems):
    _check(lib().pccl_schedule_write_direct_allreduce(_b(path), _b(dtype), _b(compute), devices, slice_elems))


def write_collective(path, kind, dtype, compute, devices, elems, root=0):
    _check(lib().pccl_schedule_write_collective(_b(path), _b(kind), _b(dtype), _b(compute), devices, elems, root))


def write_small_message(path, dtype="bf16", devices=8, n_slices=36, n_extra=64, seed=4, lo_bytes=8 << 10,
                        hi_bytes=256 << 10):
    _check(lib().pccl_schedule_write_small_message(_b(path), _b(dtype), devices, n_slices, n_extra, seed, lo_bytes, hi_bytes))


def inspect_schedule(path, want_order=True):
    n, d, e = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_long(0)
    _check(lib().pccl_schedule_inspect(_b(path), ctypes.byref(n), ctypes.byref(d), ctypes.byref(e), None, 0))
    order = None
    if want_order:
        arr = (ctypes.c_int * max(n.value, 1))()
        _check(lib().pccl_schedule_inspect(_b(path), None, None, None, arr, n.value))
        order = list(arr[:n.value])
    return {"n_ops": n.value, "devices": d.value, "elems_per_device": e.value, "order": order}
