"""ctypes binding of the CPU checker ``oracle/libpccl_oracle.so``.

TEST INFRASTRUCTURE ONLY: imported by ``tests/``, by ``__graft_entry__.smoke()`` and by
the ``cpu_baseline`` leg of ``bench.py``; never by the product package.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libpccl_oracle.so")

F32, I32, BF16, F16, F8E4M3, F8E5M2, F64, U32 = 0, 1, 2, 3, 4, 5, 6, 7
SUM, PROD, MIN, MAX = 0, 1, 2, 3
DTYPES = {"f32": F32, "i32": I32, "bf16": BF16, "f16": F16, "f8e4m3": F8E4M3, "f8e5m2": F8E5M2, "f64": F64, "u32": U32}
COMPUTES = {"sum": SUM, "prod": PROD, "min": MIN, "max": MAX}
# numpy storage type per dtype code (bf16/f16 travel as raw uint16 bit patterns)
NP_STORAGE = {F32: np.float32, I32: np.int32, BF16: np.uint16, F16: np.uint16, F8E4M3: np.uint8, F8E5M2: np.uint8,
              F64: np.float64, U32: np.uint32}


class OracleOp(ctypes.Structure):
    _fields_ = [
        ("dtype", ctypes.c_int), ("op", ctypes.c_int), ("n_in", ctypes.c_int), ("n_out", ctypes.c_int),
        ("ins", ctypes.c_void_p * 8), ("outs", ctypes.c_void_p * 8), ("count", ctypes.c_long),
    ]


def build():
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, cl, u64 = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_uint64
        L.pccl_oracle_f32_to_bf16.argtypes = [ctypes.c_float]
        L.pccl_oracle_f32_to_bf16.restype = ctypes.c_uint16
        L.pccl_oracle_f32_to_f16.argtypes = [ctypes.c_float]
        L.pccl_oracle_f32_to_f16.restype = ctypes.c_uint16
        L.pccl_oracle_bf16_to_f32.argtypes = [ctypes.c_uint16]
        L.pccl_oracle_bf16_to_f32.restype = ctypes.c_float
        L.pccl_oracle_f16_to_f32.argtypes = [ctypes.c_uint16]
        L.pccl_oracle_f16_to_f32.restype = ctypes.c_float
        L.pccl_oracle_narrow_array.argtypes = [ci, vp, vp, cl]
        L.pccl_oracle_narrow_array.restype = None
        L.pccl_oracle_widen_array.argtypes = [ci, vp, vp, cl]
        L.pccl_oracle_widen_array.restype = None
        L.pccl_oracle_narrow_array8.argtypes = [ci, vp, vp, cl]
        L.pccl_oracle_narrow_array8.restype = None
        L.pccl_oracle_widen_array8.argtypes = [ci, vp, vp, cl]
        L.pccl_oracle_widen_array8.restype = None
        L.pccl_oracle_reduce_copy.argtypes = [ci, ci, ctypes.POINTER(vp), ci, ctypes.POINTER(vp), ci, cl]
        L.pccl_oracle_reduce_copy_mt.argtypes = [ci, ci, ctypes.POINTER(vp), ci, ctypes.POINTER(vp), ci, cl, ci]
        L.pccl_oracle_run_ops.argtypes = [ctypes.POINTER(OracleOp), ci, ctypes.POINTER(ci)]
        L.pccl_oracle_topo_sort.argtypes = [ci, ctypes.POINTER(ci), ctypes.POINTER(ci), ci, ctypes.POINTER(ci)]
        L.pccl_oracle_rng_u64.argtypes = [u64, u64, u64]
        L.pccl_oracle_rng_u64.restype = u64
        L.pccl_oracle_fill_uniform_f32.argtypes = [vp, cl, u64, u64, ctypes.c_float, ctypes.c_float]
        L.pccl_oracle_fill_uniform_f32.restype = None
        L.pccl_oracle_fill_normal.argtypes = [vp, ci, cl, u64, u64, ctypes.c_double, ctypes.c_double]
        L.pccl_oracle_fill_normal.restype = None
        L.pccl_oracle_fill_normal_at.argtypes = [vp, ci, cl, cl, u64, u64, ctypes.c_double, ctypes.c_double]
        L.pccl_oracle_fill_normal_at.restype = None
        L.pccl_oracle_fill_int32.argtypes = [vp, cl, u64, u64, ctypes.c_int32, ctypes.c_int32]
        L.pccl_oracle_fill_int32.restype = None
        _lib = L
    return _lib


def _code(table, x):
    return table[x] if isinstance(x, str) else int(x)


def _ptr(a):
    return a.ctypes.data if isinstance(a, np.ndarray) else int(a)


def narrow(dtype, x):
    """float32 array -> bit patterns of bf16 / f16 (uint16) or f8e4m3 / f8e5m2 (uint8)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    dt = _code(DTYPES, dtype)
    if dt in (F8E4M3, F8E5M2):
        out = np.empty(x.shape, dtype=np.uint8)
        lib().pccl_oracle_narrow_array8(dt, x.ctypes.data, out.ctypes.data, x.size)
        return out
    out = np.empty(x.shape, dtype=np.uint16)
    lib().pccl_oracle_narrow_array(dt, x.ctypes.data, out.ctypes.data, x.size)
    return out


def widen(dtype, h):
    dt = _code(DTYPES, dtype)
    if dt in (F8E4M3, F8E5M2):
        h = np.ascontiguousarray(h, dtype=np.uint8)
        out = np.empty(h.shape, dtype=np.float32)
        lib().pccl_oracle_widen_array8(dt, h.ctypes.data, out.ctypes.data, h.size)
        return out
    h = np.ascontiguousarray(h, dtype=np.uint16)
    out = np.empty(h.shape, dtype=np.float32)
    lib().pccl_oracle_widen_array(dt, h.ctypes.data, out.ctypes.data, h.size)
    return out


def reduce_copy(dtype, compute, ins, outs, count=None, nthreads=1):
    """ins / outs: numpy arrays (or raw addresses) of the storage type; writes outs in place."""
    dt, op = _code(DTYPES, dtype), _code(COMPUTES, compute)
    if count is None:
        count = ins[0].size
    vp = ctypes.c_void_p
    a_in = (vp * max(len(ins), 1))(*[_ptr(a) for a in ins])
    a_out = (vp * max(len(outs), 1))(*[_ptr(a) for a in outs])
    if nthreads > 1:
        rc = lib().pccl_oracle_reduce_copy_mt(dt, op, a_in, len(ins), a_out, len(outs), count, nthreads)
    else:
        rc = lib().pccl_oracle_reduce_copy(dt, op, a_in, len(ins), a_out, len(outs), count)
    if rc != 0:
        raise ValueError("pccl_oracle_reduce_copy rejected its arguments")


def reduce(dtype, compute, ins):
    """Convenience: returns a fresh output array."""
    out = np.empty_like(ins[0])
    reduce_copy(dtype, compute, ins, [out])
    return out


def run_ops(ops, order=None):
    """ops: list of dicts (dtype, compute, ins, outs, count) holding numpy arrays or addresses."""
    n = len(ops)
    arr = (OracleOp * max(n, 1))()
    for i, o in enumerate(ops):
        arr[i].dtype = _code(DTYPES, o["dtype"])
        arr[i].op = _code(COMPUTES, o.get("compute", "sum"))
        arr[i].n_in, arr[i].n_out = len(o["ins"]), len(o["outs"])
        for k, a in enumerate(o["ins"]):
            arr[i].ins[k] = _ptr(a)
        for k, a in enumerate(o["outs"]):
            arr[i].outs[k] = _ptr(a)
        arr[i].count = o["count"]
    po = None
    if order is not None:
        po = (ctypes.c_int * max(n, 1))(*order)
    if lib().pccl_oracle_run_ops(arr, n, po) != 0:
        raise ValueError("pccl_oracle_run_ops rejected its arguments")


def topo_sort(n_nodes, edges):
    """edges: list of (src, dst) in insertion order.  Returns the order, or None on a cycle."""
    ne = len(edges)
    src = (ctypes.c_int * max(ne, 1))(*[e[0] for e in edges])
    dst = (ctypes.c_int * max(ne, 1))(*[e[1] for e in edges])
    out = (ctypes.c_int * max(n_nodes, 1))()
    if lib().pccl_oracle_topo_sort(n_nodes, src, dst, ne, out) != 0:
        return None
    return list(out[:n_nodes])


def rng_u64(seed, stream, index):
    return lib().pccl_oracle_rng_u64(seed, stream, index)


def fill_uniform_f32(n, seed, stream, lo, hi):
    a = np.empty(n, dtype=np.float32)
    lib().pccl_oracle_fill_uniform_f32(a.ctypes.data, n, seed, stream, lo, hi)
    return a


def fill_normal(dtype, n, seed, stream, mean=0.0, sigma=1.0, nthreads=1):
    """N(mean, sigma) values 0 .. n-1 of the stream; nthreads > 1 fills contiguous slices in parallel
    (the generator is counter-based: the same bytes either way)."""
    dt = _code(DTYPES, dtype)
    a = np.empty(n, dtype=NP_STORAGE[dt])
    if nthreads <= 1 or n < (1 << 16):
        lib().pccl_oracle_fill_normal(a.ctypes.data, dt, n, seed, stream, mean, sigma)
        return a
    from concurrent.futures import ThreadPoolExecutor
    per = (n + nthreads - 1) // nthreads
    fill = lib().pccl_oracle_fill_normal_at   # (ctypes releases the interpreter lock during the call)
    with ThreadPoolExecutor(nthreads) as pool:
        jobs = [pool.submit(fill, a.ctypes.data + lo * a.itemsize, dt, lo, min(per, n - lo), seed, stream, mean, sigma)
                for lo in range(0, n, per)]
        for j in jobs:
            j.result()
    return a


def fill_int32(n, seed, stream, lo=-(1 << 20), hi=1 << 20):
    a = np.empty(n, dtype=np.int32)
    lib().pccl_oracle_fill_int32(a.ctypes.data, n, seed, stream, lo, hi)
    return a
