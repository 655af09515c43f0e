"""ctypes binding of ``libpccl_hip.so`` (C ABI declared in ``include/pccl_hip.h``).

Operands are raw device addresses; anything with ``data_ptr()`` (a torch tensor) is
accepted in their place.  Every call raises :class:`PcclError` on a non-zero return
code, carrying the library's error text.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libpccl_hip.so")

# codes of include/pccl_hip.h
F32, I32, BF16, F16, F8E4M3, F8E5M2, F64, U32 = 0, 1, 2, 3, 4, 5, 6, 7
SUM, PROD, MIN, MAX = 0, 1, 2, 3
COPY, REDUCE, NOTIFY, GET_NOTIFIED = 0, 1, 2, 3
DTYPES = {"f32": F32, "i32": I32, "bf16": BF16, "f16": F16, "f8e4m3": F8E4M3, "f8e5m2": F8E5M2, "f64": F64, "u32": U32}
COMPUTES = {"sum": SUM, "prod": PROD, "min": MIN, "max": MAX}
ELEM_BYTES = {F32: 4, I32: 4, BF16: 2, F16: 2, F8E4M3: 1, F8E5M2: 1, F64: 8, U32: 4}

OK = 0
ERR_INVALID_ARG, ERR_UNSUPPORTED, ERR_HIP, ERR_NO_DEVICE = -1, -2, -3, -4
ERR_NOMEM, ERR_MISALIGNED, ERR_GRAPH = -5, -6, -7

MAX_INPUTS = 8
MAX_OUTPUTS = 8


class PcclError(RuntimeError):
    def __init__(self, code, text):
        super().__init__("pccl_hip error %d: %s" % (code, text))
        self.code = code


class OpDesc(ctypes.Structure):
    """struct pccl_op_desc"""
    _fields_ = [
        ("op_uid", ctypes.c_int),
        ("primitive", ctypes.c_ubyte),
        ("dtype", ctypes.c_ubyte),
        ("compute", ctypes.c_ubyte),
        ("n_in", ctypes.c_ubyte),
        ("n_out", ctypes.c_ubyte),
        ("reserved", ctypes.c_ubyte),
        ("signal_parts", ctypes.c_ushort),
        ("ins", ctypes.c_void_p * MAX_INPUTS),
        ("outs", ctypes.c_void_p * MAX_OUTPUTS),
        ("count", ctypes.c_long),
        ("n_deps", ctypes.c_int),
        ("deps", ctypes.POINTER(ctypes.c_int)),
    ]


_lib = None


def lib():
    """Loads the library on first use; no fallback when it is missing."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH, mode=ctypes.RTLD_GLOBAL)
        vp, ci, cl = ctypes.c_void_p, ctypes.c_int, ctypes.c_long
        L.pccl_hip_device_count.argtypes = [ctypes.POINTER(ci)]
        L.pccl_hip_device_info.argtypes = [ctypes.POINTER(ci), ctypes.POINTER(cl), ctypes.c_char_p, ci]
        L.pccl_hip_set_executor_id.argtypes = [ci]
        L.pccl_hip_alloc.argtypes = [ctypes.POINTER(vp), cl]
        L.pccl_hip_free.argtypes = [vp]
        L.pccl_hip_reduce_copy.argtypes = [ci, ci, ctypes.POINTER(vp), ci, ctypes.POINTER(vp), ci, cl, vp]
        L.pccl_hip_accumulate.argtypes = [ci, ci, vp, ctypes.POINTER(vp), ci, cl, vp]
        L.pccl_hip_set_tuning.argtypes = [ci, ci]
        L.pccl_hip_set_occupancy_lds.argtypes = [ci]
        L.pccl_hip_set_unroll.argtypes = [ci]
        L.pccl_hip_set_rotation.argtypes = [ci]
        L.pccl_hip_set_slice_bytes.argtypes = [cl]
        L.pccl_hip_graph_create.argtypes = [ctypes.POINTER(OpDesc), ci, cl, ctypes.POINTER(vp)]
        L.pccl_hip_graph_run_static.argtypes = [ctypes.POINTER(OpDesc), ci, cl, vp, ctypes.POINTER(ctypes.c_uint),
                                                ctypes.POINTER(ctypes.c_uint)]
        L.pccl_hip_graph_run.argtypes = [vp, vp]
        L.pccl_hip_graph_status.argtypes = [vp, vp, ctypes.POINTER(ctypes.c_uint), ctypes.POINTER(ctypes.c_uint)]
        L.pccl_hip_graph_rebind.argtypes = [vp, vp, vp, cl, vp]
        L.pccl_hip_graph_info.argtypes = [vp, ctypes.POINTER(vp), ctypes.POINTER(ci), ctypes.POINTER(ci)]
        L.pccl_hip_graph_launch_kind.argtypes = [vp, ctypes.POINTER(ci)]
        L.pccl_hip_classify_dependencies.argtypes = [ctypes.POINTER(OpDesc), ci, ctypes.POINTER(ci), vp]
        L.pccl_hip_plan_chains.argtypes = [ctypes.POINTER(OpDesc), ci, ctypes.POINTER(ci), ci, ctypes.POINTER(ci)]
        L.pccl_hip_plan_signals.argtypes = [ctypes.POINTER(OpDesc), ci, ctypes.POINTER(ci), ctypes.POINTER(ci)]
        L.pccl_hip_graph_dependency_kinds.argtypes = [vp, vp, ctypes.c_long, ctypes.POINTER(ctypes.c_long)]
        L.pccl_hip_graph_trace.argtypes = [vp, ci]
        L.pccl_hip_graph_read_trace.argtypes = [vp, vp, vp, ctypes.c_long, ctypes.POINTER(ctypes.c_long)]
        L.pccl_hip_graph_next_signal_base.argtypes = [vp, ctypes.POINTER(ctypes.c_uint)]
        L.pccl_hip_graph_set_spin_limit.argtypes = [vp, ctypes.c_uint]
        L.pccl_hip_graph_destroy.argtypes = [vp]
        for name in ("pccl_hip_last_error", "pccl_hip_version"):
            getattr(L, name).restype = ctypes.c_char_p
            getattr(L, name).argtypes = []
        _lib = L
    return _lib


def _check(rc):
    if rc != OK:
        raise PcclError(rc, lib().pccl_hip_last_error().decode())


def _addr(x):
    if x is None:
        return None
    return int(x.data_ptr()) if hasattr(x, "data_ptr") else int(x)


def _code(table, x):
    return table[x] if isinstance(x, str) else int(x)


def version():
    return lib().pccl_hip_version().decode()


def device_count():
    n = ctypes.c_int(0)
    _check(lib().pccl_hip_device_count(ctypes.byref(n)))
    return n.value


def device_info():
    cus, mem = ctypes.c_int(0), ctypes.c_long(0)
    name = ctypes.create_string_buffer(256)
    _check(lib().pccl_hip_device_info(ctypes.byref(cus), ctypes.byref(mem), name, 256))
    return {"compute_units": cus.value, "hbm_bytes": mem.value, "name": name.value.decode()}


def set_executor_id(ident):
    """The registry id the device image's executor fields carry (pccl_hip_set_executor_id)."""
    _check(lib().pccl_hip_set_executor_id(ident))


def alloc(nbytes):
    p = ctypes.c_void_p(None)
    _check(lib().pccl_hip_alloc(ctypes.byref(p), nbytes))
    return p.value


def free(ptr):
    _check(lib().pccl_hip_free(ctypes.c_void_p(ptr)))


def set_rotation(rotate=-1):
    _check(lib().pccl_hip_set_rotation(rotate))


def set_slice_bytes(nbytes=0):
    """Longest stretch of an operand that one launch covers (0: the built-in 32 GiB)."""
    _check(lib().pccl_hip_set_slice_bytes(nbytes))


def set_tuning(workgroups_per_cu=0, cache_treatment=-1):
    _check(lib().pccl_hip_set_tuning(workgroups_per_cu, cache_treatment))


def set_occupancy_lds(lds_bytes=-1):
    _check(lib().pccl_hip_set_occupancy_lds(lds_bytes))


def set_unroll(unroll=-1):
    _check(lib().pccl_hip_set_unroll(unroll))


def reduce_copy(dtype, compute, ins, outs, count, stream=None):
    """One reduce-copy launch: outs[j][:count] = fold(compute, ins[0][:count], ...)."""
    n_in, n_out = len(ins), len(outs)
    a_in = (ctypes.c_void_p * max(n_in, 1))(*[_addr(x) for x in ins])
    a_out = (ctypes.c_void_p * max(n_out, 1))(*[_addr(x) for x in outs])
    _check(lib().pccl_hip_reduce_copy(_code(DTYPES, dtype), _code(COMPUTES, compute), a_in, n_in,
                                      a_out, n_out, count, ctypes.c_void_p(_addr(stream))))


def accumulate(dtype, compute, src, outs, count, stream=None):
    """outs[j][:count] = compute(outs[j][:count], src[:count]) for every j, reading src once."""
    a_out = (ctypes.c_void_p * max(len(outs), 1))(*[_addr(x) for x in outs])
    _check(lib().pccl_hip_accumulate(_code(DTYPES, dtype), _code(COMPUTES, compute), ctypes.c_void_p(_addr(src)), a_out,
                                     len(outs), count, ctypes.c_void_p(_addr(stream))))


def _op_descs(ops):
    """list of op dicts -> (OpDesc array, objects to keep alive while it is in use)."""
    n = len(ops)
    arr = (OpDesc * max(n, 1))()
    keep = []
    for i, o in enumerate(ops):
        d = arr[i]
        d.op_uid = i
        prim = o.get("primitive")
        if prim in (NOTIFY, GET_NOTIFIED):
            # signal op: "signal" = address of the 32-bit word, "value" = 0..65535
            d.primitive = prim
            d.n_in, d.n_out = (0, 1) if prim == NOTIFY else (1, 0)
            (d.outs if prim == NOTIFY else d.ins)[0] = _addr(o["signal"])
            d.count = o["value"]
            d.signal_parts = o.get("parts", 0)   # >= 2: a signal of that many words, one per part of the data
        else:
            n_in, n_out = len(o["ins"]), len(o["outs"])
            d.primitive = prim if prim is not None else (COPY if n_in == 1 else REDUCE)
            d.dtype = _code(DTYPES, o["dtype"])
            d.compute = _code(COMPUTES, o.get("compute", "sum"))
            d.n_in, d.n_out = n_in, n_out
            for k in range(min(n_in, MAX_INPUTS)):
                d.ins[k] = _addr(o["ins"][k])
            for k in range(min(n_out, MAX_OUTPUTS)):
                d.outs[k] = _addr(o["outs"][k])
            d.count = o["count"]
        deps = list(o.get("deps", ()))
        d.n_deps = len(deps)
        buf = (ctypes.c_int * max(len(deps), 1))(*deps)
        keep.append(buf)
        d.deps = ctypes.cast(buf, ctypes.POINTER(ctypes.c_int))
    return arr, keep


def part_elems(count, parts):
    """Elements per part of an op cut into `parts` parts (the last part may be shorter)."""
    per = (count + parts - 1) // parts
    return (per + 63) // 64 * 64


def classify_dependencies(ops, parts):
    """The executor's rule for which dependencies are met part by part, without a device:
    ops as for Graph, parts[i] = number of parts of op i.  Returns one flag per dependency
    (ops in order, dependencies in list order)."""
    arr, keep = _op_descs(ops)
    n_deps = sum(len(o.get("deps", ())) for o in ops)
    kinds = (ctypes.c_ubyte * max(n_deps, 1))()
    pa = (ctypes.c_int * max(len(ops), 1))(*parts)
    _check(lib().pccl_hip_classify_dependencies(arr, len(ops), pa, kinds))
    return list(kinds)[:n_deps]


def plan_chains(ops, parts, forward_elem_bytes):
    """The executor's chain plan for these ops (host only): per op a tuple (next op or -1, ops in the
    chain it starts or 1, one-pass flag / index of the handed-on input, first row of its operand table)."""
    arr, keep = _op_descs(ops)
    pa = (ctypes.c_int * max(len(ops), 1))(*parts)
    words = (ctypes.c_int * max(4 * len(ops), 1))()
    _check(lib().pccl_hip_plan_chains(arr, len(ops), pa, forward_elem_bytes, words))
    return [tuple(words[4 * i:4 * i + 4]) for i in range(len(ops))]


def plan_signals(ops, with_parts=False):
    """Which signal ops ride on data ops (host only): per op the index of the COPY / REDUCE that carries
    it, or -1.  with_parts: also, per op, the K of a signal op carried part by part / of the data op that is
    cut into K parts for such signals (0 otherwise)."""
    arr, keep = _op_descs(ops)
    carrier = (ctypes.c_int * max(len(ops), 1))()
    parts = (ctypes.c_int * max(len(ops), 1))()
    _check(lib().pccl_hip_plan_signals(arr, len(ops), carrier, parts if with_parts else None))
    if with_parts:
        return list(carrier[:len(ops)]), list(parts[:len(ops)])
    return list(carrier[:len(ops)])


STATIC_ARENA_BYTES = 8 << 20
TILE_AUTO = -1   # graph_create: the executor chooses between the queue and plain launches


def graph_run_static(ops, stream=None, tile_bytes=0, wait=True):
    """Runs a DAG of ops with its device state in the library's fixed per-GPU array: no device
    allocation (pccl_hip_graph_run_static).  wait=True: waits for `stream` and returns
    (completed, total); wait=False: returns None once the launch is enqueued."""
    arr, keep = _op_descs(ops)
    if not wait:
        _check(lib().pccl_hip_graph_run_static(arr, len(ops), tile_bytes, ctypes.c_void_p(_addr(stream)), None, None))
        return None
    c, t = ctypes.c_uint(0), ctypes.c_uint(0)
    _check(lib().pccl_hip_graph_run_static(arr, len(ops), tile_bytes, ctypes.c_void_p(_addr(stream)), ctypes.byref(c),
                                           ctypes.byref(t)))
    del keep
    return c.value, t.value


class Graph:
    """A DAG of COPY / REDUCE ops resident on the device, drained by one launch."""

    def __init__(self, ops, tile_bytes=0):
        """ops: list of dicts with keys dtype, compute, ins, outs, count, deps (op index list)."""
        arr, self._keep = _op_descs(ops)
        self._h = ctypes.c_void_p(None)
        _check(lib().pccl_hip_graph_create(arr, len(ops), tile_bytes, ctypes.byref(self._h)))

    def run(self, stream=None):
        _check(lib().pccl_hip_graph_run(self._h, ctypes.c_void_p(_addr(stream))))

    def status(self, stream=None):
        c, t = ctypes.c_uint(0), ctypes.c_uint(0)
        _check(lib().pccl_hip_graph_status(self._h, ctypes.c_void_p(_addr(stream)), ctypes.byref(c), ctypes.byref(t)))
        return c.value, t.value

    def rebind(self, old_base, new_base, nbytes, stream=None):
        _check(lib().pccl_hip_graph_rebind(self._h, ctypes.c_void_p(_addr(old_base)), ctypes.c_void_p(_addr(new_base)),
                                           nbytes, ctypes.c_void_p(_addr(stream))))

    def next_signal_base(self):
        b = ctypes.c_uint(0)
        _check(lib().pccl_hip_graph_next_signal_base(self._h, ctypes.byref(b)))
        return b.value

    def set_spin_limit(self, microseconds):
        """How long a wait inside the kernel may last before the run gives up (default two seconds)."""
        _check(lib().pccl_hip_graph_set_spin_limit(self._h, microseconds))

    def info(self):
        lay, nt, nw = ctypes.c_void_p(None), ctypes.c_int(0), ctypes.c_int(0)
        _check(lib().pccl_hip_graph_info(self._h, ctypes.byref(lay), ctypes.byref(nt), ctypes.byref(nw)))
        return {"device_layout": lay.value, "n_tiles": nt.value, "n_workgroups": nw.value}

    def launch_kind(self):
        """'drain' (the persistent kernel), 'wide' (one workgroup per entry), 'launches' (plain launches) or 'chains'
        (a wide launch in the shape of a direct one: a few chains that are each one fold, a workgroup per 4 KiB)."""
        kind = ctypes.c_int(0)
        _check(lib().pccl_hip_graph_launch_kind(self._h, ctypes.byref(kind)))
        return ("drain", "wide", "launches", "chains")[kind.value]

    def dependency_kinds(self):
        """One flag per dependency (ops in uid order, dependencies in list order): 1 = met part
        by part, 0 = waits for the whole predecessor."""
        n = ctypes.c_long(0)
        _check(lib().pccl_hip_graph_dependency_kinds(self._h, None, 0, ctypes.byref(n)))
        buf = (ctypes.c_ubyte * max(n.value, 1))()
        _check(lib().pccl_hip_graph_dependency_kinds(self._h, buf, n.value, ctypes.byref(n)))
        return list(buf)[:n.value]

    def trace(self, enable=True):
        """Switches the per-entry timeline on or off for the following runs."""
        _check(lib().pccl_hip_graph_trace(self._h, 1 if enable else 0))

    def read_trace(self, stream=None):
        """Timeline of the last run: uint64 array (entries, 4) in queue order; columns: what
        (op_uid | part << 32 | workgroup << 52), ticket drawn, dependencies met, part complete,
        in ticks of the device's 100 MHz clock."""
        import numpy as np
        n = ctypes.c_long(0)
        _check(lib().pccl_hip_graph_read_trace(self._h, ctypes.c_void_p(_addr(stream)), None, 0, ctypes.byref(n)))
        out = np.zeros((n.value, 4), dtype=np.uint64)
        if n.value:
            _check(lib().pccl_hip_graph_read_trace(self._h, ctypes.c_void_p(_addr(stream)), out.ctypes.data_as(ctypes.c_void_p),
                                                   n.value, ctypes.byref(n)))
        return out

    def destroy(self):
        if self._h:
            _check(lib().pccl_hip_graph_destroy(self._h))
            self._h = ctypes.c_void_p(None)

    def __del__(self):
        try:
            self.destroy()
        except Exception:
            pass
