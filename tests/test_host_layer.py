"""CPU-side tests of the host layer and the C ABI surface (no GPU needed): exported symbols,
TypeRegistry, device plugins, schedule format and generators, the Python collective IR."""
import ctypes
import os
import re

import numpy as np
import pytest

import helpers as H
import schedules as S

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def E():
    from pccl_amd import engine
    engine.lib()
    return engine


def _declared(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(pccl_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported():
    from pccl_amd import hip, engine
    for header, path in (("pccl_hip.h", hip.LIB_PATH), ("pccl_engine.h", engine.LIB_PATH)):
        names = _declared(header)
        assert len(names) >= 15, names
        L = ctypes.CDLL(path, mode=ctypes.RTLD_GLOBAL)
        for n in names:
            assert hasattr(L, n), "%s declares %s but %s does not export it" % (header, n, os.path.basename(path))


def test_host_only_entry_points_answer_without_a_device():
    """The entry points that touch no device: element sizes by dtype code, the version string, the
    setters' argument checks, the error text of the calling thread."""
    from pccl_amd import hip
    L = hip.lib()
    for name, code in hip.DTYPES.items():
        assert L.pccl_hip_dtype_bytes(code) == H.ELEM_BYTES[name], name
    assert L.pccl_hip_dtype_bytes(99) == 0
    L.pccl_hip_version.restype = ctypes.c_char_p
    assert b"gfx950" in L.pccl_hip_version()
    with pytest.raises(hip.PcclError) as e:
        hip.set_slice_bytes(4097)
    assert e.value.code == hip.ERR_INVALID_ARG and "4096" in str(e.value)
    hip.set_slice_bytes(0)
    with pytest.raises(hip.PcclError):
        hip.set_rotation(5)
    with pytest.raises(hip.PcclError):
        hip.set_unroll(3)


def test_layout_header_compiles_as_c_and_matches_reference_offsets(tmp_path):
    """pccl_op_layout.h is plain C; offsets are those of the reference's operator.h / chunk.h (LP64)."""
    src = tmp_path / "t.c"
    src.write_text(r'''
#include <stdio.h>
#include "pccl_op_layout.h"
int main(void) {
  printf("%zu %zu %zu\n", sizeof(pccl_chunk_meta), offsetof(pccl_chunk_meta, addr_), offsetof(pccl_chunk_meta, num_elems_));
  printf("%zu %zu %zu %zu %zu\n", sizeof(pccl_ring_buffer), offsetof(pccl_ring_buffer, elem_size_), offsetof(pccl_ring_buffer, tail_), offsetof(pccl_ring_buffer, head_), offsetof(pccl_ring_buffer, consumer_buffer_));
  printf("%zu %zu %zu %zu %zu %zu\n", sizeof(pccl_operation_layout_header), offsetof(pccl_operation_layout_header, remaining_executors_), offsetof(pccl_operation_layout_header, pre_dependencies_), offsetof(pccl_operation_layout_header, num_next_ops_), offsetof(pccl_operation_layout_header, op_buffer_), offsetof(pccl_operation_layout_header, next_op_uids_head_));
  printf("%zu %zu %zu %zu\n", sizeof(pccl_graph_buffer_layout), offsetof(pccl_graph_buffer_layout, operators), offsetof(pccl_graph_buffer_layout, ready_queues), offsetof(pccl_graph_buffer_layout, num_queues));
  return 0;
}''')
    exe = tmp_path / "t"
    import subprocess
    subprocess.run(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout.split("\n")
    assert out[0] == "24 8 16"
    assert out[1] == "40 4 16 20 32"
    assert out[2] == "32 8 12 15 16 24"
    assert out[3] == "48 16 32 40"


# ---- TypeRegistry ------------------------------------------------------------------------------

def test_registry_plugins_registered_at_load(E):
    assert set(E.device_types()) == {"cpu", "rocm"}
    for n in ("copy", "reduce", "notify", "get_notified", "f32", "i32", "bf16", "f16", "sum", "prod", "min", "max", "hip"):
        assert E.type_name(E.type_id(n)) == n
    ids = [E.type_id(n) for n in ("cpu", "rocm", "hip", "copy", "f32", "sum")]
    assert len(set(ids)) == len(ids), "all kinds share one id space"
    for n in ("copy", "reduce", "f32", "i32", "bf16", "f16", "sum", "prod", "min", "max"):
        assert E.is_compatible("hip", n)
    assert E.is_compatible("hip", "notify") and E.is_compatible("hip", "get_notified")


def test_registry_register_and_errors(E):
    a = E.register_type("data", "test_dtype_x")
    assert E.register_type("data", "test_dtype_x") == a, "same name, same id"
    b = E.register_type("compute", "test_compute_y")
    assert b == a + 1, "one shared counter"
    with pytest.raises(E.EngineError):
        E.register_type("device", "test_dtype_x")  # already a data type
    with pytest.raises(E.EngineError):
        E.type_id("no_such_type")
    with pytest.raises(E.EngineError):
        E.type_name(250)
    with pytest.raises(E.EngineError):
        E.register_compatibility("no_such_executor", "f32")
    with pytest.raises(E.EngineError):
        E.register_compatibility("hip", "no_such_type")
    E.register_compatibility("hip", "test_dtype_x")
    assert E.is_compatible("hip", "test_dtype_x")


# ---- device plugins ----------------------------------------------------------------------------

def test_cpu_plugin_allocator(E):
    assert E.allocator_available("cpu")
    assert not E.ipc_available("cpu") and not E.ipc_available("rocm")
    p = E.allocate("cpu", 1 << 20)
    assert p
    buf = (ctypes.c_ubyte * (1 << 20)).from_address(p)
    buf[0], buf[(1 << 20) - 1] = 7, 9
    assert (buf[0], buf[(1 << 20) - 1]) == (7, 9)
    E.deallocate("cpu", p)
    assert E.allocate("cpu", 0) is None and E.allocate("cpu", -5) is None
    with pytest.raises(E.EngineError):
        E.allocator_available("hip")  # an executor, not a device


def test_launch_options_listed(E):
    assert {"PCCL_HIP_WG_PER_CU", "PCCL_HIP_NT", "PCCL_HIP_TILE_BYTES"} <= set(E.LaunchEnvironments.listOpt())
    E.LaunchEnvironments.registerOpt("PCCL_TEST_OPTION")
    E.LaunchEnvironments.registerOpt("PCCL_TEST_OPTION")
    assert E.LaunchEnvironments.listOpt().count("PCCL_TEST_OPTION") == 1
    assert E.LaunchEnvironments.getEnv("PCCL_SURELY_UNSET_VARIABLE") == ""
    assert E.LaunchEnvironments.getEnv("PATH") == os.environ["PATH"]


# ---- schedules ----------------------------------------------------------------------------------

def test_native_and_python_emitters_agree(E, tmp_path):
    from pccl_amd import lang
    p = str(tmp_path / "a.sched")
    E.write_small_message(p)
    ir, per = lang.small_message_allreduce()
    assert open(p).read() == ir.serialize(per)
    for world, n, dt, op in ((8, 1000, "f32", "max"), (2, 5, "bf16", "sum"), (3, 77, "i32", "prod"), (1, 4, "f16", "min")):
        E.write_ring_allreduce(p, dt, op, world, n)
        ir, per = lang.ring_allreduce(world, n, dt, op)
        assert open(p).read() == ir.serialize(per)
        for kind, emit in (("ring_allreduce", lambda: lang.ring_allreduce(world, n, dt, op)),
                           ("direct_allreduce", lambda: lang.direct_allreduce(world, n, dt, op)),
                           ("ring_reduce_scatter", lambda: lang.ring_reduce_scatter(world, n, dt, op)),
                           ("ring_all_gather", lambda: lang.ring_all_gather(world, n, dt)),
                           ("all_to_all", lambda: lang.all_to_all(world, n, dt)),
                           ("broadcast", lambda: lang.broadcast(world, n, root=world - 1, dtype=dt))):
            E.write_collective(p, kind, dt, op if kind not in ("ring_all_gather", "broadcast", "all_to_all") else "sum", world, n, world - 1)
            ir, per = emit()
            assert open(p).read() == ir.serialize(per), kind
    with pytest.raises(E.EngineError):
        E.write_collective(p, "all_to_some", "f32", "sum", 4, 8)


def test_schedule_order_matches_reference_rule(E, oracle, tmp_path):
    """Schedule::topologicalOrder, the Python DirectedGraph and the CPU checker's restatement of
    pccl/lang/utils/graph.py:94-112 give the same order, and it respects every dependency."""
    from pccl_amd import lang
    p = str(tmp_path / "a.sched")
    E.write_small_message(p, n_slices=3, n_extra=5)
    info = E.inspect_schedule(p)
    hdr, ops = S.parse_schedule_text(open(p).read())
    assert info["n_ops"] == len(ops) == 3 * 112 + 5 and info["devices"] == 8
    assert info["order"] == oracle.topo_sort(len(ops), S.edges_of(ops))
    ir, _ = lang.small_message_allreduce(n_slices=3, n_extra=5)
    assert info["order"] == [o.op_id for o in ir.get_operation_sequence()]
    pos = {op: i for i, op in enumerate(info["order"])}
    assert all(pos[d] < pos[i] for i, o in enumerate(ops) for d in o["deps"])


def _replay_ir(oracle, ir, per, dtype, host_in):
    """Runs a Python-emitted schedule on the CPU checker: returns the "out" buffers of all ranks."""
    hdr, ops = S.parse_schedule_text(ir.serialize(per))
    W = hdr["devices"]
    out = np.zeros(W * per, dtype=H.STORAGE[dtype])
    bufs = {"in": host_in, "out": out}
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs[b][r * per + e:r * per + e + n]), order)
    return out.reshape(W, per)


def test_python_collectives_compute_what_they_say(E, oracle, tmp_path):
    """reduce-scatter, all-gather, direct all-reduce and broadcast emitters, replayed on the CPU
    checker and compared with their definitions in numpy terms."""
    from pccl_amd import lang
    W, n = 5, 37
    x = H.gen("f32", W * W * n, 60, 0).reshape(W, W * n)          # rank r's "in": W chunks of n
    flat = x.reshape(-1)
    # reduce-scatter: rank r ends with chunk (r+1) mod W folded around the ring from the chunk's own rank
    ir, per = lang.ring_reduce_scatter(W, n, "f32", "sum")
    out = _replay_ir(oracle, ir, per, "f32", flat)
    for r in range(W):
        c = (r + 1) % W
        acc = x[c, c * n:(c + 1) * n].copy()
        for i in range(1, W):
            acc = (x[(c + i) % W, c * n:(c + 1) * n] + acc).astype(np.float32)     # incoming first, then own
        H.assert_bits_equal(out[r, c * n:(c + 1) * n], acc, "reduce-scatter rank %d" % r)
    # all-gather: every rank's out = concatenation of chunk r of rank r
    ir, per = lang.ring_all_gather(W, n, "f32")
    out = _replay_ir(oracle, ir, per, "f32", flat)
    want = np.concatenate([x[r, r * n:(r + 1) * n] for r in range(W)])
    for r in range(W):
        H.assert_bits_equal(out[r], want, "all-gather rank %d" % r)
    # direct all-reduce: every rank's out = fold over ranks 0..W-1 in that order; same text as the native generator
    ir, per = lang.direct_allreduce(W, n, "f32", "sum")
    out = _replay_ir(oracle, ir, per, "f32", flat)
    want = oracle.reduce("f32", "sum", [x[r].copy() for r in range(W)])
    for r in range(W):
        H.assert_bits_equal(out[r], want, "direct all-reduce rank %d" % r)
    p = str(tmp_path / "d.sched")
    for world in (1, 2, 8):
        E.write_direct_allreduce(p, "f32", "sum", world, n)
        ir, per = lang.direct_allreduce(world, n, "f32", "sum")
        assert open(p).read().replace("name direct_allreduce_%d" % world, "name direct_allreduce") == ir.serialize(per) \
            or open(p).read().split("\n", 2)[2] == ir.serialize(per).split("\n", 2)[2]
    # all-to-all: out[d] chunk r = in[r] chunk d
    ir, per = lang.all_to_all(W, n, "f32")
    out = _replay_ir(oracle, ir, per, "f32", flat)
    for d in range(W):
        for r in range(W):
            H.assert_bits_equal(out[d, r * n:(r + 1) * n], x[r, d * n:(d + 1) * n], "all-to-all %d <- %d" % (d, r))
    # broadcast from rank 3
    ir, per = lang.broadcast(W, 3 * n, root=3, dtype="f32")
    out = _replay_ir(oracle, ir, per, "f32", x[:, :3 * n].copy().reshape(-1))
    for r in range(W):
        H.assert_bits_equal(out[r], x[3, :3 * n], "broadcast rank %d" % r)
    with pytest.raises(ValueError):
        lang.direct_allreduce(9, 4)
    # element sizes of every dtype name
    for dt, es in lang.ELEM_BYTES.items():
        ir, per = lang.small_message_allreduce(world=2, n_slices=2, n_extra=1, lo_bytes=64, hi_bytes=128, dtype=dt)
        assert 64 // es <= per


def test_direct_allreduce_schedule_shape(E, tmp_path):
    p = str(tmp_path / "d.sched")
    E.write_direct_allreduce(p, "bf16", "sum", 8, 4096)
    hdr, ops = S.parse_schedule_text(open(p).read())
    assert hdr["elems_per_device"] == 8 * 4096 and len(ops) == 16
    red, bc = ops[0], ops[1]
    assert [x[1] for x in red["ins"]] == list(range(8)) and len(red["outs"]) == 1
    assert len(bc["ins"]) == 1 and len(bc["outs"]) == 7 and bc["deps"] == [0]


@pytest.mark.parametrize("text, why", [
    ("pccl-schedule 3\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 0\n", "version"),
    ("pccl-schedule 2\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 NOTIFY 4 deps 0 slot 3\n", "expected parts"),
    ("pccl-schedule 2\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 NOTIFY 4 deps 0 slot 250 parts 8\n", "does not fit"),
    ("pccl-schedule 2\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 GET_NOTIFIED 4 deps 0 slot 0 parts 0\n", "parts out of range"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 NOTIFY 4 deps 0 slot 3 parts 2\n", "trailing text"),
    ("pccl-schedule 1\nname x\ndtype q7\ncompute sum\ndevices 1\nelems_per_device 4\nops 0\n", "dtype"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute xor\ndevices 1\nelems_per_device 4\nops 0\n", "compute"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 NOTIFY 4 deps 0 slot 256\n", "signal slot"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 GET_NOTIFIED 70000 deps 0 slot 3\n", "signal value"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 NOTIFY 4 deps 0 src 1 in 0 0 dst 1 out 0 0\n", "expected 'slot'"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 COPY 8 deps 0 src 1 in 0 0 dst 1 out 0 0\n", "past elems_per_device"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 COPY 4 deps 0 src 1 in 0 0 dst 1 in 0 0\n", "read-only"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 2\n"
     "op 0 COPY 4 deps 1 1 src 1 in 0 0 dst 1 out 0 0\nop 1 COPY 4 deps 1 0 src 1 in 0 0 dst 1 out 0 0\n", "cycle"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n"
     "op 0 COPY 4 deps 0 src 2 in 0 0 in 0 0 dst 1 out 0 0\n", "one source"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 2\nelems_per_device 4\nops 1\n"
     "op 0 COPY 4 deps 0 src 1 in 2 0 dst 1 out 0 0\n", "device"),
    ("pccl-schedule 1\nname x\ndtype f32\ncompute sum\ndevices 1\nelems_per_device 4\nops 1\n", "end of file"),
])
def test_schedule_parser_rejects(E, text, why):
    eng = E.Engine(0, 1)
    eng.initEngine()
    with pytest.raises(E.EngineError) as e:
        eng.regOpText("bad", text)
    assert why.lower() in str(e.value).lower(), str(e.value)
    eng.close()


def test_schedule_format_version_2_says_signals_of_a_slot_per_part(E, tmp_path):
    """A signalled ring whose signals take K slots, one per part of the chunk they announce, is written as
    "pccl-schedule 2" with "parts K" behind every signal op's slot; the native parser loads it (and version 1
    files as before), and the same ring with one-slot signals is still written as version 1."""
    from pccl_amd import lang
    ir, per = lang.ring_allreduce_signalled(4, 1000, dtype="f32", first_slot=8, signal_parts=4)
    text = ir.serialize(per)
    assert text.startswith("pccl-schedule 2\n")
    hdr, ops = S.parse_schedule_text(text)
    sig = [o for o in ops if o.get("signal")]
    assert hdr["version"] == 2 and len(sig) == 44 and all(o["parts"] == 4 for o in sig)
    assert sorted(set(o["slot"] for o in sig)) == [8, 12, 16, 20]          # link r: slots 8 + 4 r ...
    p = str(tmp_path / "v2.sched")
    ir.save(p, per)
    assert E.inspect_schedule(p, want_order=False)["n_ops"] == len(ops)
    eng = E.Engine(0, 1)
    eng.initEngine()
    eng.regOp("v2", p)
    assert eng.opInfo("v2")["n_ops"] == len(ops)
    eng.close()
    plain, _ = lang.ring_allreduce_signalled(4, 1000, dtype="f32", first_slot=8)
    assert plain.serialize(per).startswith("pccl-schedule 1\n") and " parts " not in plain.serialize(per)
    with pytest.raises(ValueError):
        lang.ring_allreduce_signalled(8, 1000, signal_parts=33)            # 8 links x 33 slots > 256


def test_engine_without_gpu_fails_loudly(E, tmp_path):
    """On a box without a GPU the engine initialises (cpu workspace only), registers schedules, and
    exeOp raises instead of computing anything on the CPU."""
    import torch
    if torch.cuda.is_available():
        pytest.skip("this check is for boxes without a GPU")
    eng = E.Engine(0, 1)
    eng.initEngine()
    ws, sig, nbytes = eng.getDevBuffer("cpu")
    assert nbytes == 1 << 28 and sig == ws + (1 << 28)
    with pytest.raises(E.EngineError):
        eng.getDevBuffer("rocm")
    p = str(tmp_path / "r.sched")
    E.write_ring_allreduce(p, "f32", "sum", 2, 16)
    eng.regOp("ar", p)
    assert eng.opInfo("ar") == {"n_ops": 4, "devices": 2, "elems_per_device": 32, "elem_bytes": 4}
    a, b = torch.zeros(64), torch.zeros(64)
    with pytest.raises(E.EngineError):
        eng.exeOp("ar", a, b)
    with pytest.raises(E.EngineError):
        eng.exeOp("unknown_name", a, b)
    for call in (eng.exportEndpoint, eng.exitCluster, lambda: eng.joinCluster("127.0.0.1:1")):
        with pytest.raises(E.EngineError) as e:
            call()
        assert "control plane" in str(e.value)
    with pytest.raises(E.EngineError):
        E.Engine(3, 2)
    eng.close()


# ---- Python collective IR (reference pccl/lang) -----------------------------------------------------

def test_directed_graph_follows_reference_rules():
    from pccl_amd.lang import DirectedGraph
    g = DirectedGraph()
    assert [g.add_node(data=100 + i) for i in range(4)] == [0, 1, 2, 3]  # ids are dense; data is not the id
    with pytest.raises(ValueError):
        g.add_edge(0, 4)
    for e in ((0, 1), (0, 2), (1, 3), (2, 3)):
        g.add_edge(*e)
    assert g.get_successors(0) == [1, 2] and g.get_predecessors(3) == [1, 2]
    assert g.is_acyclic() and g.topological_sort() == [0, 2, 1, 3]
    g.add_edge(3, 0)
    assert not g.is_acyclic()
    with pytest.raises(ValueError):
        g.topological_sort()
    g.remove_edge(3, 0)
    assert g.is_acyclic()
    h = DirectedGraph()
    for _ in range(5):
        h.add_node()
    h.add_edge(0, 1)
    h.add_edge(3, 4)
    assert sorted(map(sorted, h.get_connected_components())) == [[0, 1], [2], [3, 4]]
    deep = DirectedGraph()
    for i in range(5000):  # deeper than the interpreter's recursion limit
        deep.add_node()
        if i:
            deep.add_edge(i - 1, i)
    assert deep.topological_sort() == list(range(5000))


def test_collective_ir_container():
    from pccl_amd.lang import Chunk, CollectiveIR, Device, DeviceType, Link, PrimitiveOpType
    ir = CollectiveIR("t", dtype="f32")
    for d in range(3):
        ir.add_device(Device(d, DeviceType.ROCM, 8e12, 9.5))
    with pytest.raises(ValueError):
        ir.add_device(Device(7, DeviceType.ROCM, 8e12, 9.5))  # ids must be dense, in order
    ir.add_link(Link(0, 1, 1e11, 1e-6))
    assert not ir.validate_topology()
    ir.add_link(Link(1, 2, 1e11, 1e-6))
    assert ir.validate_topology()
    assert ir.get_device_bandwidth_matrix()[(2, 1)] == 1e11
    c = Chunk({0}, 0, 16, 0)
    c2 = c.copy()
    c2.reduced_ranks.add(1)
    assert c.reduced_ranks == {0}
    a = ir.create_operation(PrimitiveOpType.COPY, c, Chunk({0}, 1, 16, 0), 0, 1)
    b = ir.create_operation(PrimitiveOpType.REDUCE, Chunk({0}, 1, 16, 0), Chunk({0, 2}, 2, 16, 0), 1, 2, dependencies=[a])
    assert (a, b) == (0, 1) and ir.validate_dag()
    assert [o.op_id for o in ir.get_operation_sequence()] == [0, 1]
    low = ir.lower()
    assert low[1]["ins"] == [("out", 1, 0), ("out", 2, 0)] and low[1]["outs"] == [("out", 2, 0)]  # reduce src into tgt
    ir.create_operation(PrimitiveOpType.NOTIFY, c, c, 0, 1)
    with pytest.raises(ValueError):
        ir.lower()  # a signal op needs a slot and a value
    ir.ops[2].metadata.update(slot=5, value=9)
    w = ir.create_operation(PrimitiveOpType.GET_NOTIFIED, c, c, 0, 1, dependencies=[b], metadata=dict(slot=5, value=9))
    low = ir.lower()
    assert low[2]["primitive"] == 2 and low[w]["primitive"] == 3 and low[w]["slot"] == 5 and low[w]["deps"] == [b]
    text = ir.serialize()
    assert "op 2 NOTIFY 9 deps 0 slot 5" in text and "op 3 GET_NOTIFIED 9 deps 1 1 slot 5" in text
    bad = CollectiveIR("cyc")
    x = bad.create_operation(PrimitiveOpType.COPY, c, c, 0, 0)
    bad.op_dag.add_edge(x, x)
    assert not bad.validate_dag() and bad.get_operation_sequence() == []


def test_extension_module_has_the_reference_layout(E, tmp_path):
    """pccl_amd.engine_c is a compiled extension module laid out like the reference's pccl.engine_c
    (csrc/python_api.cc:13-27): class Engine with the reference's methods, submodule utils with
    LaunchEnvironments; it shares the registry and the option list with the C ABI's view."""
    import torch  # noqa: F401  (a torch extension: torch's libraries and type casters come first)
    from pccl_amd import engine_c
    assert engine_c.__file__.endswith(".so")
    for method in ("initEngine", "regOp", "exeOp", "exportEndpoint", "joinCluster", "exitCluster"):
        assert callable(getattr(engine_c.Engine, method))
    assert engine_c.utils.LaunchEnvironments.listOpt() == E.LaunchEnvironments.listOpt()
    assert engine_c.utils.LaunchEnvironments.getEnv("PATH") == os.environ["PATH"]
    eng = engine_c.Engine(0, 1)
    for call in (eng.exportEndpoint, lambda: eng.joinCluster("127.0.0.1:1"), eng.exitCluster):
        with pytest.raises(RuntimeError, match="no cluster control plane"):
            call()
    with pytest.raises(RuntimeError, match="open file"):
        eng.regOp("ring", str(tmp_path / "missing.sched"))
    with pytest.raises(RuntimeError):
        engine_c.Engine(3, 2)            # rank outside the world
    # tensors that are not on the device are refused before anything is launched
    eng2 = engine_c.Engine(0, 1)
    x = torch.zeros(16)
    with pytest.raises(RuntimeError):
        eng2.exeOp("nothing", x, x.clone())


def test_tensor_overload_header_compiles_against_torch(tmp_path):
    """engine_torch.h gives Engine::exeOp the reference's at::Tensor signature (include/engine.h:19);
    it is header-only, so the check is that it compiles against this image's torch headers."""
    import subprocess
    from torch.utils import cpp_extension
    src = tmp_path / "t.cc"
    src.write_text('#include "engine_torch.h"\n'
                   'void run(engine_c::TorchEngine &e, at::Tensor &a, at::Tensor b) { e.exeOp("op", a, b); }\n'
                   'void run2(engine_c::Engine &e, at::Tensor &a, at::Tensor b) { engine_c::exeOp(e, "op", a, b); }\n')
    cmd = ["g++", "-std=c++17", "-fsyntax-only", "-D__HIP_PLATFORM_AMD__", "-I/opt/rocm/include",
           "-I", os.path.join(ROOT, "pccl_amd", "csrc", "host"), "-I", os.path.join(ROOT, "include")]
    for inc in cpp_extension.include_paths():
        cmd += ["-I", inc]
    subprocess.run(cmd + [str(src)], check=True)


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits with status 2 before
    touching torch or the GPU."""
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 2
    assert "one GPU" in r.stderr and r.stdout.strip() == ""


def test_product_uses_neither_the_checker_nor_working_files():
    """The CPU checker under oracle/ is test infrastructure: nothing in the package or the public
    headers may import, link or name it (or the builder's scratch folder); only tests/, smoke() and
    the CPU-baseline leg of bench.py do."""
    bad = []
    pattern = re.compile(r"\boracle\b|\b_work\b|pccl_oracle")
    for top in ("pccl_amd", "include"):
        for folder, _, files in os.walk(os.path.join(ROOT, top)):
            if "__pycache__" in folder or os.path.join("csrc", "build") in folder:
                continue
            for name in files:
                if not name.endswith((".py", ".cc", ".h", ".hip", "Makefile")):
                    continue
                path = os.path.join(folder, name)
                for n, line in enumerate(open(path, errors="replace"), 1):
                    if pattern.search(line):
                        bad.append("%s:%d: %s" % (os.path.relpath(path, ROOT), n, line.strip()))
    assert not bad, "\n".join(bad)
    # bench.py reaches the checker in its CPU-baseline leg only
    lines = open(os.path.join(ROOT, "bench.py")).read().split("\n")
    uses = [n for n, line in enumerate(lines) if re.search(r"\boracle\b", line) and not line.lstrip().startswith("#")]
    start = next(n for n, line in enumerate(lines) if line.startswith("def cpu_baseline"))
    end = next(n for n in range(start + 1, len(lines)) if lines[n].startswith("def "))
    assert uses and all(start <= n < end for n in uses), [lines[n] for n in uses if not start <= n < end]
