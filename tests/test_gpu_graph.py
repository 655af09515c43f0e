"""GPU parity of the op-batching path: DAGs drained by one persistent kernel (C ABI
pccl_hip_graph_*) against the CPU checker executing the same ops in topological order."""
import ctypes

import numpy as np
import pytest

import helpers as H
import schedules as S

pytestmark = pytest.mark.gpu


def _stream(torch):
    return torch.cuda.current_stream().cuda_stream


def _run_and_check(torch, hip, g, n_ops):
    g.run(_stream(torch))
    done, total = g.status(_stream(torch))
    assert (done, total) == (n_ops, n_ops)


def test_single_op_graph(hip, oracle):
    import torch
    for dtype, count in (("bf16", 32768), ("f32", 70001), ("i32", 5), ("f16", 1 << 20), ("f64", 50001), ("u32", 7777)):
        ins = [H.gen(dtype, count, 31, k) for k in range(2)]
        want = oracle.reduce(dtype, "sum", ins)
        d_in = [H.DevBuf(torch, dtype, count, 0, src=a) for a in ins]
        d_out = H.DevBuf(torch, dtype, count, 0)
        g = hip.Graph([dict(dtype=dtype, compute="sum", ins=[b.ptr for b in d_in], outs=[d_out.ptr], count=count)])
        _run_and_check(torch, hip, g, 1)
        H.assert_bits_equal(d_out.download(), want, "single-op graph %s" % dtype)
        assert d_out.guards_intact()
        g.destroy()


def test_dependent_chain_in_place(hip, oracle):
    """t = a+b; u = t+c; t = u+t (in place); v = copy(t) -- wrong order gives wrong bits."""
    import torch
    count = 200003
    a, b, c = (H.gen("f32", count, 41, k, kind="uniform", lo=-1e3, hi=1e3) for k in range(3))
    t = oracle.reduce("f32", "sum", [a, b])
    u = oracle.reduce("f32", "sum", [t, c])
    t2 = oracle.reduce("f32", "sum", [u, t])
    da, db, dc = (H.DevBuf(torch, "f32", count, 4 * k, src=x) for k, x in enumerate((a, b, c)))
    dt, du, dv = (H.DevBuf(torch, "f32", count, 8 * k) for k in range(3))
    ops = [
        dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
        dict(dtype="f32", compute="sum", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[0]),
        dict(dtype="f32", compute="sum", ins=[du.ptr, dt.ptr], outs=[dt.ptr], count=count, deps=[1]),
        dict(dtype="f32", compute="sum", ins=[dt.ptr], outs=[dv.ptr], count=count, deps=[2]),
    ]
    g = hip.Graph(ops, tile_bytes=16384)
    assert g.info()["n_tiles"] > 4
    _run_and_check(torch, hip, g, 4)
    H.assert_bits_equal(du.download(), u, "u")
    H.assert_bits_equal(dt.download(), t2, "t (in place)")
    H.assert_bits_equal(dv.download(), t2, "v (copy)")
    g.destroy()


def _ring_case(torch, hip, oracle, world, sizes, dtype, seed, offsets=(0, 0), tile_bytes=0, runs=1):
    es = H.ELEM_BYTES[dtype]
    ops, per_rank = S.ring_allreduce_ops(world, sizes, dtype=dtype)
    host_in = [H.gen(dtype, per_rank, seed, r, sigma=1.0) for r in range(world)]
    host_out = [np.zeros(per_rank, dtype=H.STORAGE[dtype]) for _ in range(world)]
    # CPU checker: same ops, order restated from the reference's topological_sort
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    assert order is not None
    bufs = {"in": host_in, "out": host_out}
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs[b][r][e:e + n]), order)
    # every rank ends with the same bytes: the all-reduce invariant
    for r in range(1, world):
        H.assert_bits_equal(host_out[r], host_out[0], "oracle: rank %d vs rank 0" % r)
    d_in = [H.DevBuf(torch, dtype, per_rank, offsets[0], src=host_in[r]) for r in range(world)]
    d_out = [H.DevBuf(torch, dtype, per_rank, offsets[1]) for r in range(world)]
    dev = {"in": d_in, "out": d_out}
    g = hip.Graph(S.materialise(ops, lambda b, r, e, n: dev[b][r].ptr + e * es), tile_bytes=tile_bytes)
    for it in range(runs):
        if it:
            for b in d_out:
                b.view().fill_(0xFF)
        _run_and_check(torch, hip, g, len(ops))
        for r in range(world):
            H.assert_bits_equal(d_out[r].download(), host_out[r], "run %d rank %d" % (it, r))
            assert d_out[r].guards_intact()
    info = g.info()
    g.destroy()
    return info


def test_ring_allreduce_small(hip, oracle):
    import torch
    _ring_case(torch, hip, oracle, 8, [1000, 37, 4096], "bf16", seed=4)


def test_ring_allreduce_world_sizes(hip, oracle):
    import torch
    for world in (2, 3, 5, 8):
        _ring_case(torch, hip, oracle, world, [2049, 64], "f32", seed=5)


def test_ring_allreduce_unaligned_and_rerun(hip, oracle):
    """Operands 6 and 10 bytes off 16-byte alignment; graph run three times (self re-arming)."""
    import torch
    _ring_case(torch, hip, oracle, 8, [5001, 12345, 3], "bf16", seed=6, offsets=(6, 10), tile_bytes=4096, runs=3)


def test_config5_shape_reduced(hip, oracle):
    """The 4096-op construction at reduced byte sizes: 36 ring slices x 112 ops + 64 copies."""
    import torch
    sizes = S.log_uniform_sizes(oracle, 36, 4, 0, 512, 16384, 2)
    world = 8
    ops, per_rank = S.ring_allreduce_ops(world, sizes, dtype="bf16")
    extra = S.log_uniform_sizes(oracle, 64, 4, 1, 512, 16384, 2)
    off = per_rank
    for i, n in enumerate(extra):  # 64 independent level-1 copies, 8 per rank
        r = i % world
        ops.append(dict(dtype="bf16", compute="sum", ins=[("in", r, off)], outs=[("out", r, off)], count=n, deps=[]))
        if r == world - 1:
            off += max(extra[i - 7:i + 1])
    per_rank = off + max(extra)
    assert len(ops) == 4096
    host_in = [H.gen("bf16", per_rank, 4, 10 + r, sigma=1.0) for r in range(world)]
    host_out = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    bufs = {"in": host_in, "out": host_out}
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs[b][r][e:e + n]), order)
    d_in = [H.DevBuf(torch, "bf16", per_rank, 0, src=host_in[r]) for r in range(world)]
    d_out = [H.DevBuf(torch, "bf16", per_rank, 0, fill=0) for r in range(world)]
    dev = {"in": d_in, "out": d_out}
    g = hip.Graph(S.materialise(ops, lambda b, r, e, n: dev[b][r].ptr + e * 2))
    for it in range(2):
        _run_and_check(torch, hip, g, 4096)
        for r in range(world):
            H.assert_bits_equal(d_out[r].download(), host_out[r], "run %d rank %d" % (it, r))
    g.destroy()


def test_rebind(hip, oracle):
    import torch
    count = 40000
    a, b, a2 = (H.gen("bf16", count, 51, k) for k in range(3))
    da, db, da2 = (H.DevBuf(torch, "bf16", count, 0, src=x) for x in (a, b, a2))
    do, do2 = H.DevBuf(torch, "bf16", count, 0), H.DevBuf(torch, "bf16", count, 0)
    g = hip.Graph([dict(dtype="bf16", compute="sum", ins=[da.ptr, db.ptr], outs=[do.ptr], count=count)])
    _run_and_check(torch, hip, g, 1)
    H.assert_bits_equal(do.download(), oracle.reduce("bf16", "sum", [a, b]), "before rebind")
    g.rebind(da.ptr, da2.ptr, da.nbytes, _stream(torch))
    g.rebind(do.ptr, do2.ptr, do.nbytes, _stream(torch))
    _run_and_check(torch, hip, g, 1)
    H.assert_bits_equal(do2.download(), oracle.reduce("bf16", "sum", [a2, b]), "after rebind")
    g.destroy()


def test_graph_errors(hip):
    import torch
    t = torch.zeros(4096, dtype=torch.float32, device="cuda")
    op = dict(dtype="f32", compute="sum", ins=[t, t], outs=[t], count=16, deps=[])
    with pytest.raises(hip.PcclError) as e:  # cycle
        hip.Graph([dict(op, deps=[1]), dict(op, deps=[0])])
    assert e.value.code == hip.ERR_GRAPH
    with pytest.raises(hip.PcclError) as e:  # dependency outside the graph
        hip.Graph([dict(op, deps=[5])])
    assert e.value.code == hip.ERR_GRAPH
    with pytest.raises(hip.PcclError) as e:  # self dependency
        hip.Graph([dict(op, deps=[0])])
    assert e.value.code == hip.ERR_GRAPH
    with pytest.raises(hip.PcclError) as e:  # unknown primitive code
        hip.Graph([dict(op, primitive=9)])
    assert e.value.code == hip.ERR_UNSUPPORTED
    with pytest.raises(hip.PcclError) as e:
        hip.Graph([dict(op, ins=[t.data_ptr() + 1, t])])
    assert e.value.code == hip.ERR_MISALIGNED
    g = hip.Graph([])  # empty graph runs and reports 0 of 0
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (0, 0)
    g.destroy()


def test_bounded_wait_aborts_cleanly(hip, oracle):
    """A dependency that is never satisfied (forced from the host by inflating one op's
    pre_dependencies_ on the device) must end in PCCL_ERR_GRAPH, not in a hang, and the
    graph must work again afterwards."""
    import torch
    count = 1024
    a, b = H.gen("f32", count, 61, 0), H.gen("f32", count, 61, 1)
    da, db = H.DevBuf(torch, "f32", count, 0, src=a), H.DevBuf(torch, "f32", count, 0, src=b)
    dt, du, dv = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    # (op 0 has two successors, so that op 1 waits for it through the queue instead of running
    # behind it in the same workgroup)
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
           dict(dtype="f32", compute="sum", ins=[dt.ptr, db.ptr], outs=[du.ptr], count=count, deps=[0]),
           dict(dtype="f32", ins=[dt.ptr], outs=[dv.ptr], count=count, deps=[0])]
    g = hip.Graph(ops)
    g.set_spin_limit(20000)  # microseconds
    # GraphBufferLayout.operators (offset 16) -> headers; op 1's byte 12 is pre_dependencies_
    lay = g.info()["device_layout"]
    host = torch.empty(48, dtype=torch.uint8)
    import ctypes as C
    hipmemcpy = C.CDLL("libamdhip64.so").hipMemcpy
    hipmemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]
    assert hipmemcpy(host.data_ptr(), lay, 48, 2) == 0
    operators = int(host.numpy()[16:24].view(np.uint64)[0])
    ptrs = torch.empty(16, dtype=torch.uint8)
    assert hipmemcpy(ptrs.data_ptr(), operators, 16, 2) == 0
    hdr1 = int(ptrs.numpy()[8:16].view(np.uint64)[0])
    two = torch.tensor([2], dtype=torch.uint8)
    assert hipmemcpy(hdr1 + 12, two.data_ptr(), 1, 1) == 0  # needs 2 predecessors, has 1
    g.run(_stream(torch))
    with pytest.raises(hip.PcclError) as e:
        g.status(_stream(torch))
    assert e.value.code == hip.ERR_GRAPH
    # status restored the pristine graph: it runs correctly now
    g.set_spin_limit(2000000)
    _run_and_check(torch, hip, g, 3)
    H.assert_bits_equal(du.download(), oracle.reduce("f32", "sum", [oracle.reduce("f32", "sum", [a, b]), b]), "after reset")
    g.destroy()


def test_device_image_carries_the_executor_id(hip):
    """RingBuffer::producer_ / consumer_ (include/base/operator.h:8-9) and OperationLayoutHeader::executor_type_
    (:24), read back through the reference's offsets, hold the id given to pccl_hip_set_executor_id (the host
    layer passes the registry id of "hip")."""
    import ctypes as C
    import torch
    hipmemcpy = C.CDLL("libamdhip64.so").hipMemcpy
    hipmemcpy.argtypes = [C.c_void_p, C.c_void_p, C.c_size_t, C.c_int]

    def read(addr, n):
        host = torch.empty(n, dtype=torch.uint8)
        assert hipmemcpy(host.data_ptr(), addr, n, 2) == 0
        return host.numpy()

    x, y = H.DevBuf(torch, "f32", 4096, 0), H.DevBuf(torch, "f32", 4096, 0)
    ops = [dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=4096, deps=[])]
    try:
        from pccl_amd import engine
        for ident in (0, 37, engine.type_id("hip")):
            hip.set_executor_id(ident)
            g = hip.Graph(ops)
            layout = read(g.info()["device_layout"], 48)
            operators = int(layout[16:24].view(np.uint64)[0])
            queues = int(layout[32:40].view(np.uint64)[0])
            assert int(layout[24:28].view(np.uint32)[0]) == 1 and int(layout[40:44].view(np.uint32)[0]) == 8
            header = read(int(read(operators, 8).view(np.uint64)[0]), 32)
            assert header[13] == ident, "executor_type_"
            ring = read(int(read(queues, 8).view(np.uint64)[0]), 40)
            assert ring[0] == ident and ring[1] == ident, "producer_ / consumer_"
            g.destroy()
        with pytest.raises(hip.PcclError):
            hip.set_executor_id(256)
    finally:
        # what the host layer sets when it registers its executor (loading it does that)
        from pccl_amd import engine
        hip.set_executor_id(engine.type_id("hip"))


# ---- signal ops: NOTIFY / GET_NOTIFIED ---------------------------------------------------------

def _signal_ring_ops(world, size, signals_ptr, dev_in, dev_out, es=2, dtype="bf16"):
    """Ring all-reduce written the way ranks on different GPUs would have to write it: DAG edges
    only inside a rank; the hand-over between ranks goes NOTIFY (producer rank) -> signal word ->
    GET_NOTIFIED (consumer rank).  Signal word of link p -> r: slot r; value: the step number.
    Returns (ops, data_ops) where data_ops maps op index -> symbolic op for the CPU replay."""
    ops, sym = [], {}
    last_of_rank = {}           # rank -> its latest op (program order inside a rank)
    notify_of = {}              # (rank, step) -> index of the NOTIFY that publishes that step's output

    def add(op):
        ops.append(op)
        return len(ops) - 1

    for step in range(1, 2 * world - 1):
        reduce_phase = step < world
        for r in range(world):
            p = (r - 1) % world
            c = (r - step) % world if reduce_phase else (r - (step - (world - 1)) + 1) % world
            deps = [last_of_rank[r]] if r in last_of_rank else []
            if step > 1:  # wait for the neighbour's previous step through the signal word of link p -> r
                w = add(dict(primitive=3, signal=signals_ptr + 4 * r, value=step - 1, deps=deps))
                deps = [w]
            off = c * size
            if reduce_phase:
                src = ("in" if step == 1 else "out", p, off)
                o = dict(dtype=dtype, compute="sum", ins=[src, ("in", r, off)], outs=[("out", r, off)], count=size, deps=deps)
            else:
                o = dict(dtype=dtype, compute="sum", ins=[("out", p, off)], outs=[("out", r, off)], count=size, deps=deps)
            bound = dict(o)
            bound["ins"] = [(dev_in if b == "in" else dev_out)[rk].ptr + e * es for (b, rk, e) in o["ins"]]
            bound["outs"] = [(dev_in if b == "in" else dev_out)[rk].ptr + e * es for (b, rk, e) in o["outs"]]
            i = add(bound)
            sym[i] = o
            # tell the next rank that this step's output is there: link r -> r+1 is slot r+1
            n = add(dict(primitive=2, signal=signals_ptr + 4 * ((r + 1) % world), value=step, deps=[i]))
            notify_of[(r, step)] = n
            last_of_rank[r] = n
    return ops, sym


@pytest.mark.parametrize("size,tile,own_rounds", [(3001, 0, None), (30001, 8192, "16"), (30001, 8192, "0")])
def test_ring_allreduce_over_signal_words(hip, oracle, monkeypatch, size, tile, own_rounds):
    """(Second and third case: more entries than workgroups.  The entries of this graph wait for each other,
    so they are drawn by ticket whatever PCCL_HIP_OWN_ENTRIES allows.)"""
    import torch
    if own_rounds is not None:
        monkeypatch.setenv("PCCL_HIP_OWN_ENTRIES", own_rounds)
    world = 8
    per = world * size
    host_in = [H.gen("bf16", per, 81 + it, 0) for it in range(2)]  # two runs, different inputs
    d_in = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    d_out = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    signals = torch.zeros(64, dtype=torch.int32, device="cuda")
    ops, sym = _signal_ring_ops(world, size, signals.data_ptr(), d_in, d_out)
    assert sum(1 for o in ops if o.get("primitive") == 2) == world * (2 * world - 2)
    g = hip.Graph(ops, tile_bytes=tile)
    assert tile == 0 or g.info()["n_tiles"] > g.info()["n_workgroups"]
    # CPU replay of the data ops: program order of creation is a valid order
    for it in range(2):
        ins = [H.gen("bf16", per, 90 + 10 * it, r) for r in range(world)]
        outs = [np.zeros(per, dtype=np.uint16) for _ in range(world)]
        bufs = {"in": ins, "out": outs}
        for i in sorted(sym):
            o = sym[i]
            oracle.reduce_copy("bf16", "sum", [bufs[b][r][e:e + size] for (b, r, e) in o["ins"]],
                               [bufs[b][r][e:e + size] for (b, r, e) in o["outs"]])
        for r in range(world):
            d_in[r].upload(ins[r])
            d_out[r].view().fill_(0xFF)
        base = g.next_signal_base()
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (len(ops), len(ops))
        for r in range(world):
            H.assert_bits_equal(d_out[r].download(), outs[r], "run %d rank %d" % (it, r))
        # every link's word ends at the last step of this run
        assert signals[:world].cpu().tolist() == [base + 2 * world - 2] * world
    g.destroy()


def test_get_notified_from_outside_and_never(hip, oracle):
    """A wait satisfied by a word the host set before the launch passes; a wait nobody satisfies
    ends in PCCL_ERR_GRAPH through the bounded wait (no hang), and the graph works afterwards."""
    import torch
    count = 2048
    a = H.gen("f32", count, 85, 0)
    da, do = H.DevBuf(torch, "f32", count, 0, src=a), H.DevBuf(torch, "f32", count, 0)
    sig = torch.zeros(4, dtype=torch.int32, device="cuda")
    ops = [dict(primitive=3, signal=sig.data_ptr(), value=7, deps=[]),
           dict(dtype="f32", compute="sum", ins=[da.ptr], outs=[do.ptr], count=count, deps=[0])]
    g = hip.Graph(ops)
    g.set_spin_limit(20000)  # microseconds
    base = g.next_signal_base()
    sig[0] = base + 7 - (1 << 32) if base + 7 >= (1 << 31) else base + 7
    torch.cuda.synchronize()
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (2, 2)
    H.assert_bits_equal(do.download(), a, "copy released by an outside notify")
    # next run: the word still holds the previous run's value, which must NOT satisfy the wait
    do.view().fill_(0)
    g.run(_stream(torch))
    with pytest.raises(hip.PcclError) as e:
        g.status(_stream(torch))
    assert e.value.code == hip.ERR_GRAPH
    assert int(do.view().max()) == 0, "the dependent copy must not have run"
    # the aborted run still consumed a run number; set the word for the coming one and run again
    sig[0] = g.next_signal_base() + 7
    torch.cuda.synchronize()
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (2, 2)
    H.assert_bits_equal(do.download(), a, "after the aborted run")
    g.destroy()


def test_signal_op_argument_errors(hip):
    import torch
    sig = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(hip.PcclError) as e:
        hip.Graph([dict(primitive=2, signal=sig.data_ptr() + 2, value=1)])
    assert e.value.code == hip.ERR_MISALIGNED
    with pytest.raises(hip.PcclError) as e:
        hip.Graph([dict(primitive=2, signal=sig.data_ptr(), value=70000)])
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.Graph([dict(primitive=3, signal=0, value=1)])
    assert e.value.code == hip.ERR_INVALID_ARG
    # a wait that depends on the very notify that would satisfy it, in reverse: cycle through the signal
    with pytest.raises(hip.PcclError) as e:
        hip.Graph([dict(primitive=3, signal=sig.data_ptr(), value=1, deps=[]),
                   dict(primitive=2, signal=sig.data_ptr(), value=1, deps=[0])])
    assert e.value.code == hip.ERR_GRAPH


def test_copy_ops_keep_their_own_element_size(hip, oracle):
    """COPY ops of 4-byte and 2-byte elements inside graphs whose REDUCE ops use the other size
    (and in copy-only graphs): byte counts come from the op's dtype, not from the graph's kernel."""
    import torch
    n = 70001
    f = H.gen("f32", n, 95, 0)
    b = H.gen("bf16", n, 95, 1)
    df, dfo = H.DevBuf(torch, "f32", n, 4, src=f), H.DevBuf(torch, "f32", n, 12)
    db, dbo = H.DevBuf(torch, "bf16", n, 2, src=b), H.DevBuf(torch, "bf16", n, 6)
    dsum = H.DevBuf(torch, "bf16", n, 0)
    cases = {
        "copy-only": [dict(dtype="f32", compute="sum", ins=[df.ptr], outs=[dfo.ptr], count=n),
                      dict(dtype="bf16", compute="sum", ins=[db.ptr], outs=[dbo.ptr], count=n)],
        "bf16 reduce + f32 copy": [dict(dtype="bf16", compute="sum", ins=[db.ptr, db.ptr], outs=[dsum.ptr], count=n),
                                   dict(dtype="f32", compute="sum", ins=[df.ptr], outs=[dfo.ptr], count=n),
                                   dict(dtype="bf16", compute="sum", ins=[dsum.ptr], outs=[dbo.ptr], count=n, deps=[0])],
    }
    for name, ops in cases.items():
        for buf in (dfo, dbo, dsum):
            buf.view().fill_(0xFF)
        g = hip.Graph(ops, tile_bytes=8192)
        _run_and_check(torch, hip, g, len(ops))
        H.assert_bits_equal(dfo.download(), f, name + ": f32 copy")
        want_b = b if name == "copy-only" else oracle.reduce("bf16", "sum", [b, b])
        H.assert_bits_equal(dbo.download(), want_b, name + ": bf16 copy")
        assert dfo.guards_intact() and dbo.guards_intact()
        g.destroy()


def test_mixed_dtypes_and_computes_in_one_graph(hip, oracle):
    """REDUCE ops of different (dtype, compute) pairs in one graph run the kernel instance that
    picks the fold per part.  The f16 product overflows to infinity and the f8 sums saturate:
    both depend on the same hardware mode bit, which that instance switches per part; small
    parts make workgroups alternate between the two."""
    import torch
    n = 100_003
    s = _stream(torch)
    def dev(dtype, a, off=0):
        return H.DevBuf(torch, dtype, n, off, src=a)
    specs = [("bf16", "sum", 3, {}), ("f32", "max", 2, {}), ("f16", "prod", 4, dict(mean=0.0, sigma=40.0)),
             ("f8e4m3", "sum", 4, dict(sigma=200.0)), ("i32", "min", 5, {}), ("f64", "sum", 2, {}),
             ("u32", "max", 3, {}), ("f8e5m2", "prod", 3, dict(sigma=300.0)), ("f16", "sum", 8, dict(sigma=3e4))]
    ops, checks = [], []
    for k, (dtype, compute, n_in, kw) in enumerate(specs):
        ins = [H.gen(dtype, n, 500 + k, j, **kw) for j in range(n_in)]
        d_in = [dev(dtype, a, (2 * j * H.ELEM_BYTES[dtype]) % 16 if k % 2 else 0) for j, a in enumerate(ins)]
        d_out = H.DevBuf(torch, dtype, n, 0)
        ops.append(dict(dtype=dtype, compute=compute, ins=[b.ptr for b in d_in], outs=[d_out.ptr], count=n))
        checks.append((dtype, compute, d_out, oracle.reduce(dtype, compute, ins), d_in))
    # a dependent pair across dtypes' instances: copy of the f32 result, then f32 sum with itself
    f32_out = checks[1][2]
    cp, tw = H.DevBuf(torch, "f32", n, 4), H.DevBuf(torch, "f32", n, 0)
    ops.append(dict(dtype="f32", compute="sum", ins=[f32_out.ptr], outs=[cp.ptr], count=n, deps=[1]))
    ops.append(dict(dtype="f32", compute="sum", ins=[cp.ptr, f32_out.ptr], outs=[tw.ptr], count=n, deps=[len(ops) - 1]))
    g = hip.Graph(ops, tile_bytes=8192)
    for it in range(2):
        for _, _, d_out, _, _ in checks:
            d_out.view().fill_(0xFF)
        _run_and_check(torch, hip, g, len(ops))
        for dtype, compute, d_out, want, _ in checks:
            got = d_out.download()
            if dtype.startswith("f8") or dtype == "f16":
                nan_w, nan_g = np.isnan(oracle.widen(dtype, want)), np.isnan(oracle.widen(dtype, got))
                assert np.array_equal(nan_w, nan_g), "%s %s NaN positions" % (dtype, compute)
                got, want = np.where(nan_w, 0, got), np.where(nan_w, 0, want)
            H.assert_bits_equal(got, want, "run %d %s %s" % (it, dtype, compute))
            assert d_out.guards_intact()
        H.assert_bits_equal(cp.download(), checks[1][3], "copy")
        H.assert_bits_equal(tw.download(), oracle.reduce("f32", "sum", [checks[1][3], checks[1][3]]), "sum after copy")
    # the f16 cases did overflow to infinity and the f8 cases did saturate
    assert np.isinf(oracle.widen("f16", checks[2][3])).any() and np.isinf(oracle.widen("f16", checks[8][3])).any()
    assert (checks[3][3] & 0x7f == 0x7e).any() and (checks[7][3] & 0x7f == 0x7b).any()
    g.destroy()


# ---- per-entry timeline -------------------------------------------------------------------

def test_trace_records_every_entry_once_and_in_dependency_order(hip, oracle):
    """The timeline of a run names every (op, part) exactly once, its three times are ordered,
    and no part of an op starts before the parts it needs of its dependencies are done."""
    import torch
    count = 100000  # 200 KB of bf16: several parts per op
    a, b, c = (H.gen("bf16", count, 91, k) for k in range(3))
    da, db, dc = (H.DevBuf(torch, "bf16", count, 0, src=x) for x in (a, b, c))
    dt, du, dv = (H.DevBuf(torch, "bf16", count, 0) for _ in range(3))
    ops = [dict(dtype="bf16", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
           dict(dtype="bf16", compute="max", ins=[db.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[]),
           dict(dtype="bf16", compute="sum", ins=[dt.ptr, du.ptr], outs=[dv.ptr], count=count, deps=[0, 1])]
    g = hip.Graph(ops)
    with pytest.raises(hip.PcclError):
        g.read_trace(_stream(torch))  # never switched on
    g.trace(True)
    for _ in range(2):  # each run overwrites the last
        _run_and_check(torch, hip, g, 3)
    tr = g.read_trace(_stream(torch))
    info = g.info()
    assert tr.shape == (info["n_tiles"], 4)
    uid = (tr[:, 0] & np.uint64(0xffffffff)).astype(np.int64)
    part = ((tr[:, 0] >> np.uint64(32)) & np.uint64(0xfffff)).astype(np.int64)
    wg = (tr[:, 0] >> np.uint64(52)).astype(np.int64)
    assert wg.min() >= 0 and wg.max() < info["n_workgroups"]
    for u in range(3):
        assert sorted(part[uid == u].tolist()) == list(range(int((uid == u).sum()))) and (uid == u).sum() > 1
    claimed, ready, done = (tr[:, k].astype(np.int64) for k in (1, 2, 3))
    assert (claimed > 0).all() and (claimed <= ready).all() and (ready <= done).all()
    # op 2 reads what ops 0 and 1 wrote, at the same addresses and cut alike: its part p needs
    # their parts p (not the whole ops)
    for p in range(int((uid == 2).sum())):
        mine = ready[(uid == 2) & (part == p)][0]
        assert mine >= done[(uid == 0) & (part == p)][0] and mine >= done[(uid == 1) & (part == p)][0]
    assert done.max() - claimed.min() < 100 * 1000 * 100  # under 100 ms of the 100 MHz clock
    want = oracle.reduce("bf16", "sum", [oracle.reduce("bf16", "sum", [a, b]), oracle.reduce("bf16", "max", [b, c])])
    H.assert_bits_equal(dv.download(), want, "traced run")
    # switched off: runs still work and leave the records alone
    g.trace(False)
    _run_and_check(torch, hip, g, 3)
    assert np.array_equal(g.read_trace(_stream(torch)), tr)
    g.destroy()


# ---- dependencies met part by part ---------------------------------------------------------

def _timeline(torch, g):
    tr = g.read_trace(_stream(torch))
    uid = (tr[:, 0] & np.uint64(0xffffffff)).astype(np.int64)
    part = ((tr[:, 0] >> np.uint64(32)) & np.uint64(0xfffff)).astype(np.int64)
    return uid, part, tr[:, 2].astype(np.int64), tr[:, 3].astype(np.int64)


def test_chain_of_large_in_place_ops_streams_part_by_part(hip, oracle, monkeypatch):
    """t = a + b; t = t * c (in place); u = max(t, a); t = u + t: every op has many parts and
    reads or overwrites its predecessor's output at the same addresses, so part p follows
    part p.  Bits must equal the ops executed one after the other.  (With every op queueing its
    own entries, which is what the timeline shows; tests/test_gpu_chains.py covers the same ops
    with op 1 running behind op 0 in one workgroup.)"""
    import torch
    monkeypatch.setenv("PCCL_HIP_CHAINS", "0")
    count = 3 * 1000 * 1000 + 17
    a, b, c = (H.gen("f32", count, 97, k) for k in range(3))
    da, db, dc = (H.DevBuf(torch, "f32", count, 0, src=x) for x in (a, b, c))
    dt, du = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
           dict(dtype="f32", compute="prod", ins=[dt.ptr, dc.ptr], outs=[dt.ptr], count=count, deps=[0]),
           dict(dtype="f32", compute="max", ins=[dt.ptr, da.ptr], outs=[du.ptr], count=count, deps=[1]),
           dict(dtype="f32", compute="sum", ins=[du.ptr, dt.ptr], outs=[dt.ptr], count=count, deps=[2, 1])]
    g = hip.Graph(ops)
    g.trace(True)
    t1 = oracle.reduce("f32", "prod", [oracle.reduce("f32", "sum", [a, b]), c])
    u = oracle.reduce("f32", "max", [t1, a])
    want = oracle.reduce("f32", "sum", [u, t1])
    for _ in range(3):
        _run_and_check(torch, hip, g, 4)
        H.assert_bits_equal(dt.download(), want, "chain t")
        H.assert_bits_equal(du.download(), u, "chain u")
    uid, part, ready, done = _timeline(torch, g)
    n_parts = int((uid == 0).sum())
    assert n_parts > 16 and all(int((uid == k).sum()) == n_parts for k in range(4))
    for k in (1, 2, 3):  # part p never before part p of the op before
        for p in range(n_parts):
            assert ready[(uid == k) & (part == p)][0] >= done[(uid == k - 1) & (part == p)][0]
    # ... and the chain did overlap: some part of op 1 was ready before op 0 was complete
    assert ready[uid == 1].min() < done[uid == 0].max()
    assert dt.guards_intact() and du.guards_intact()
    g.destroy()


def test_shifted_overlap_keeps_the_dependency_whole(hip, oracle):
    """B reads A's output 64 elements further on (and, behind A, X's output likewise): part p
    of B needs other parts of A, so B must wait for all of A.  Checked on the timeline and on
    the bits."""
    import torch
    count, shift = 2 * 1000 * 1000, 64
    a, b = H.gen("bf16", count, 98, 0), H.gen("bf16", count, 98, 1)
    tail = H.gen("bf16", shift, 98, 2)
    da, db = H.DevBuf(torch, "bf16", count, 0, src=a), H.DevBuf(torch, "bf16", count, 0, src=b)
    dT = H.DevBuf(torch, "bf16", count + shift, 0, src=np.concatenate([np.zeros(count, dtype=tail.dtype), tail]))
    dU, dV, dW = (H.DevBuf(torch, "bf16", count, 0) for _ in range(3))
    es = 2
    ops = [  # X: T[0:n] = a + b
           dict(dtype="bf16", compute="sum", ins=[da.ptr, db.ptr], outs=[dT.ptr], count=count, deps=[]),
           # A: U = T[0:n] + a           (same addresses as X's output: part by part)
           dict(dtype="bf16", compute="sum", ins=[dT.ptr, da.ptr], outs=[dU.ptr], count=count, deps=[0]),
           # B: V = U + T[64:n+64]       (U at A's addresses, but T shifted against X, which lies behind A)
           dict(dtype="bf16", compute="sum", ins=[dU.ptr, dT.ptr + shift * es], outs=[dV.ptr], count=count, deps=[1]),
           # C: W = T[64:n+64] + b       (shifted against X directly)
           dict(dtype="bf16", compute="sum", ins=[dT.ptr + shift * es, db.ptr], outs=[dW.ptr], count=count, deps=[0])]
    g = hip.Graph(ops)
    g.trace(True)
    T = np.concatenate([oracle.reduce("bf16", "sum", [a, b]), tail])
    U = oracle.reduce("bf16", "sum", [T[:count], a])
    for _ in range(3):
        _run_and_check(torch, hip, g, 4)
        H.assert_bits_equal(dU.download(), U, "U")
        H.assert_bits_equal(dV.download(), oracle.reduce("bf16", "sum", [U, T[shift:]]), "V")
        H.assert_bits_equal(dW.download(), oracle.reduce("bf16", "sum", [T[shift:], b]), "W")
    uid, part, ready, done = _timeline(torch, g)
    assert ready[uid == 2].min() >= done[uid == 1].max()  # B after all of A (hence all of X)
    assert ready[uid == 3].min() >= done[uid == 0].max()  # C after all of X
    g.destroy()


def test_rebind_that_changes_aliasing_rebuilds_the_graph(hip, oracle, monkeypatch):
    """A: t = a + b; B: u = t + c.  Rebinding u onto a's buffer, shifted, makes B overwrite what
    A reads: the dependency turns whole-op (graph rebuilt inside rebind); rebinding it back
    restores the part-by-part form.  Results must match sequential execution each time."""
    import torch
    monkeypatch.setenv("PCCL_HIP_WIDE", "0")  # (as a wide launch the graph would refuse that rebind: see the test below)
    count, shift = 1500 * 1000, 64
    a_full = H.gen("f32", count + shift, 99, 0)
    b, c = H.gen("f32", count, 99, 1), H.gen("f32", count, 99, 2)
    dA = H.DevBuf(torch, "f32", count + shift, 0, src=a_full)
    db, dc = H.DevBuf(torch, "f32", count, 0, src=b), H.DevBuf(torch, "f32", count, 0, src=c)
    dt, du = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    ops = [dict(dtype="f32", compute="sum", ins=[dA.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
           dict(dtype="f32", compute="sum", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[0])]
    g = hip.Graph(ops)
    g.trace(True)
    t = oracle.reduce("f32", "sum", [a_full[:count], b])
    u = oracle.reduce("f32", "sum", [t, c])
    _run_and_check(torch, hip, g, 2)
    H.assert_bits_equal(du.download(), u, "before rebind")
    uid, part, ready, done = _timeline(torch, g)
    assert all(ready[(uid == 1) & (part == p)][0] >= done[(uid == 0) & (part == p)][0] for p in range(int((uid == 1).sum())))
    # u -> a's buffer + 64 elements
    g.rebind(du.ptr, dA.ptr + 4 * shift, 4 * count, _stream(torch))
    g.trace(True)
    for _ in range(2):
        dA.upload(a_full)
        _run_and_check(torch, hip, g, 2)
        H.assert_bits_equal(dt.download(), t, "t after rebind")
        got = dA.download()
        H.assert_bits_equal(got[shift:], u, "u inside a's buffer")
        H.assert_bits_equal(got[:shift], a_full[:shift], "a's first elements")
        uid, part, ready, done = _timeline(torch, g)
        assert ready[uid == 1].min() >= done[uid == 0].max()
    # and back
    g.rebind(dA.ptr + 4 * shift, du.ptr, 4 * count, _stream(torch))
    dA.upload(a_full)
    du.upload(np.zeros(count, dtype=np.float32).view(u.dtype))
    _run_and_check(torch, hip, g, 2)
    H.assert_bits_equal(du.download(), u, "after rebinding back")
    assert dA.guards_intact() and du.guards_intact() and dt.guards_intact()
    g.destroy()


def test_wide_launch_refuses_a_rebind_that_makes_an_entry_wait(hip, oracle):
    """The same two ops with the library's own choices: B runs behind A in A's workgroups, no entry waits
    for another, so the graph runs as a wide launch (one workgroup per entry, more than the device holds
    at once).  The rebind that makes B wait for all of A cannot be carried out by such a launch: it is
    refused before anything changes, the graph goes on with the operands it had, and other rebinds work."""
    import torch
    count, shift = 6 * 1000 * 1000, 64
    a_full = H.gen("f32", count + shift, 199, 0)
    b, c = H.gen("f32", count, 199, 1), H.gen("f32", count, 199, 2)
    dA = H.DevBuf(torch, "f32", count + shift, 0, src=a_full)
    db, dc = H.DevBuf(torch, "f32", count, 0, src=b), H.DevBuf(torch, "f32", count, 0, src=c)
    dt, du, dv = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    g = hip.Graph([dict(dtype="f32", compute="sum", ins=[dA.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
                   dict(dtype="f32", compute="sum", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[0])])
    info = g.info()
    assert g.launch_kind() == "wide"
    assert info["n_workgroups"] == info["n_tiles"] == (4 * count + 8191) // 8192, info  # one workgroup per 8 KiB block of the chain
    t = oracle.reduce("f32", "sum", [a_full[:count], b])
    u = oracle.reduce("f32", "sum", [t, c])
    for _ in range(2):
        _run_and_check(torch, hip, g, 2)
        H.assert_bits_equal(du.download(), u, "wide launch")
        H.assert_bits_equal(dt.download(), t, "t")
    with pytest.raises(hip.PcclError) as e:
        g.rebind(du.ptr, dA.ptr + 4 * shift, 4 * count, _stream(torch))
    assert e.value.code == hip.ERR_UNSUPPORTED and "wide launch" in str(e.value)
    du.upload(np.zeros(count, dtype=np.float32).view(u.dtype))
    _run_and_check(torch, hip, g, 2)
    H.assert_bits_equal(du.download(), u, "after the refused rebind")
    g.rebind(du.ptr, dv.ptr, 4 * count, _stream(torch))  # (a move that keeps the plan)
    _run_and_check(torch, hip, g, 2)
    H.assert_bits_equal(dv.download(), u, "after a rebind that keeps the plan")
    assert all(d.guards_intact() for d in (dA, dt, du, dv))
    g.destroy()


def test_wide_launch_and_persistent_drain_leave_the_same_bytes(hip, oracle, monkeypatch):
    """Independent ops of ragged sizes and odd alignments, a chain that runs in one pass, and a fold of
    three inputs with a copy of its output that the fold stores itself: as a wide launch, with a
    timeline, and through the persistent drain (PCCL_HIP_WIDE=0)."""
    import torch
    rng = np.random.default_rng(5)
    def build():
        ops, checks = [], []
        for k in range(12):  # independent ops
            n_in, count = int(rng.integers(1, 6)), int(rng.integers(1, 70000))
            srcs = [H.gen("bf16", count, 300 + k, j) for j in range(n_in)]
            ds = [H.DevBuf(torch, "bf16", count, int(rng.integers(0, 8)) * 2, src=x) for x in srcs]
            do = H.DevBuf(torch, "bf16", count, int(rng.integers(0, 8)) * 2)
            ops.append(dict(dtype="bf16", compute="sum", ins=[d.ptr for d in ds], outs=[do.ptr], count=count, deps=[]))
            checks.append((do, oracle.reduce("bf16", "sum", srcs), ds))
        count = 150001
        x = [H.gen("bf16", count, 340, j) for j in range(5)]
        dx = [H.DevBuf(torch, "bf16", count, 0, src=v) for v in x]
        d1, d2, d3, d4 = (H.DevBuf(torch, "bf16", count, 0) for _ in range(4))
        base = len(ops)
        # a chain that runs in one pass
        ops.append(dict(dtype="bf16", compute="sum", ins=[dx[0].ptr, dx[1].ptr], outs=[d1.ptr], count=count, deps=[]))
        ops.append(dict(dtype="bf16", compute="sum", ins=[d1.ptr, dx[2].ptr], outs=[d2.ptr], count=count, deps=[base]))
        r1 = oracle.reduce("bf16", "sum", [x[0], x[1]])
        r2 = oracle.reduce("bf16", "sum", [r1, x[2]])
        # three inputs (through memory), then a copy of the result, which the fold stores itself
        ops.append(dict(dtype="bf16", compute="sum", ins=[dx[2].ptr, dx[3].ptr, dx[4].ptr], outs=[d3.ptr], count=count, deps=[]))
        ops.append(dict(dtype="bf16", compute="sum", ins=[d3.ptr], outs=[d4.ptr], count=count, deps=[base + 2]))
        r3 = oracle.reduce("bf16", "sum", [x[2], x[3], x[4]])
        checks += [(d1, r1, dx), (d2, r2, []), (d3, r3, []), (d4, r3, [])]
        return ops, checks
    ops, checks = build()
    g = hip.Graph(ops)
    info = g.info()
    assert g.launch_kind() == "wide" and info["n_workgroups"] == info["n_tiles"], info
    g.trace(True)
    for _ in range(2):
        for do, _, _ in checks: do.upload(np.zeros(do.count, dtype=np.uint16))
        _run_and_check(torch, hip, g, len(ops))
        for k, (do, want, _) in enumerate(checks):
            H.assert_bits_equal(do.download(), want, "wide launch, output %d" % k)
            assert do.guards_intact()
    uid, part, ready, done = _timeline(torch, g)
    assert len(uid) == info["n_tiles"] and (done >= ready).all()
    g.destroy()
    monkeypatch.setenv("PCCL_HIP_WIDE", "0")
    g = hip.Graph(ops)
    info = g.info()
    assert g.launch_kind() == "drain" and info["n_workgroups"] <= 4096 and info["n_workgroups"] <= info["n_tiles"]
    for do, _, _ in checks: do.upload(np.zeros(do.count, dtype=np.uint16))
    _run_and_check(torch, hip, g, len(ops))
    for k, (do, want, _) in enumerate(checks):
        H.assert_bits_equal(do.download(), want, "persistent drain, output %d" % k)
    g.destroy()


def test_part_dependencies_can_be_switched_off(hip, oracle, monkeypatch):
    import torch
    monkeypatch.setenv("PCCL_HIP_PART_DEPS", "0")
    count = 1000 * 1000
    a, b = H.gen("bf16", count, 100, 0), H.gen("bf16", count, 100, 1)
    da, db = H.DevBuf(torch, "bf16", count, 0, src=a), H.DevBuf(torch, "bf16", count, 0, src=b)
    dt, du = H.DevBuf(torch, "bf16", count, 0), H.DevBuf(torch, "bf16", count, 0)
    g = hip.Graph([dict(dtype="bf16", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
                   dict(dtype="bf16", compute="sum", ins=[dt.ptr, db.ptr], outs=[du.ptr], count=count, deps=[0])])
    g.trace(True)
    _run_and_check(torch, hip, g, 2)
    uid, part, ready, done = _timeline(torch, g)
    assert ready[uid == 1].min() >= done[uid == 0].max()
    H.assert_bits_equal(du.download(), oracle.reduce("bf16", "sum", [oracle.reduce("bf16", "sum", [a, b]), b]), "whole-op")
    g.destroy()


def test_rebind_refuses_a_move_that_breaks_element_alignment(hip, oracle):
    """f64 operands moved by 4 bytes: refused, and the graph keeps working where it was."""
    import torch
    count = 5000
    a, b = H.gen("f64", count, 101, 0), H.gen("f64", count, 101, 1)
    da, db = H.DevBuf(torch, "f64", count, 0, src=a), H.DevBuf(torch, "f64", count, 0, src=b)
    do, spare = H.DevBuf(torch, "f64", count, 0), H.DevBuf(torch, "f64", count + 1, 0)
    g = hip.Graph([dict(dtype="f64", compute="sum", ins=[da.ptr, db.ptr], outs=[do.ptr], count=count)])
    with pytest.raises(hip.PcclError) as e:
        g.rebind(do.ptr, spare.ptr + 4, 8 * count, _stream(torch))
    assert e.value.code == hip.ERR_MISALIGNED
    _run_and_check(torch, hip, g, 1)
    H.assert_bits_equal(do.download(), oracle.reduce("f64", "sum", [a, b]), "after the refused rebind")
    g.rebind(do.ptr, spare.ptr + 8, 8 * count, _stream(torch))
    _run_and_check(torch, hip, g, 1)
    H.assert_bits_equal(spare.download()[1:], oracle.reduce("f64", "sum", [a, b]), "after the good rebind")
    assert spare.guards_intact()
    g.destroy()


@pytest.mark.parametrize("block,last_level", [("1", "1"), ("3", "1"), ("32", "1"), ("0", "1"), ("3", "0")])
def test_ops_of_a_level_take_turns_in_blocks_of_parts(hip, oracle, monkeypatch, block, last_level):
    """Three chains of two many-part ops each (the second reads and overwrites what the first
    wrote, part by part) plus a single-part op: whatever the number of consecutive parts an op
    contributes to the queue order before the next op of its level takes its turn, the bits are
    those of the ops executed one after the other, and the order recorded by the timeline is
    the blocked one; the last level goes op after op, longest parts first (PCCL_HIP_LAST_LEVEL=0:
    in blocks like the others)."""
    import torch
    monkeypatch.setenv("PCCL_HIP_ORDER_BLOCK", block)
    monkeypatch.setenv("PCCL_HIP_LAST_LEVEL", last_level)
    monkeypatch.setenv("PCCL_HIP_CHAINS", "0")  # every op queues its own entries: the order of those is the subject
    counts = [700 * 1000 + 3, 300 * 1000, 1000 * 1000 + 11]
    ops, want, outs = [], [], []
    for c, count in enumerate(counts):
        a, b = H.gen("bf16", count, 120 + c, 0), H.gen("bf16", count, 120 + c, 1)
        da, db = H.DevBuf(torch, "bf16", count, 0, src=a), H.DevBuf(torch, "bf16", count, 0, src=b)
        dt = H.DevBuf(torch, "bf16", count, 0)
        outs.append((da, db, dt))
        ops.append(dict(dtype="bf16", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]))
        t = oracle.reduce("bf16", "sum", [a, b])
        want.append(oracle.reduce("bf16", "max", [t, b]))
    for c, count in enumerate(counts):
        da, db, dt = outs[c]
        ops.append(dict(dtype="bf16", compute="max", ins=[dt.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[c]))
    small = H.gen("bf16", 100, 130, 0)
    ds, dso = H.DevBuf(torch, "bf16", 100, 0, src=small), H.DevBuf(torch, "bf16", 100, 0)
    ops.append(dict(dtype="bf16", compute="sum", ins=[ds.ptr], outs=[dso.ptr], count=100, deps=[]))
    g = hip.Graph(ops, tile_bytes=16 << 10)
    g.trace(True)
    for _ in range(3):  # the graph re-arms itself, part words included
        _run_and_check(torch, hip, g, len(ops))
        for c in range(len(counts)):
            H.assert_bits_equal(outs[c][2].download(), want[c], "chain %d, block %s" % (c, block))
        H.assert_bits_equal(dso.download(), small, "single-part op")
    uid, part, ready, done = _timeline(torch, g)
    # level 0 holds ops 0, 1, 2 and 6, level 1 ops 3, 4, 5; inside a level the ops take turns
    # with `block` consecutive parts each
    n_parts = {u: int(part[uid == u].max()) + 1 for u in range(len(ops))}
    assert all(n_parts[c] == n_parts[3 + c] and n_parts[c] > 8 for c in range(3)) and n_parts[6] == 1
    expect = []
    for level_ops in ((0, 1, 2, 6), (3, 4, 5)):
        # (ops 3, 4, 5 move the same bytes per part: "longest first" leaves them in their order)
        b = 1 << 30 if level_ops[0] == 3 and last_level == "1" else (int(block) or 1 << 30)
        most = max(n_parts[u] for u in level_ops)
        for first in range(0, most, b):
            for u in level_ops:
                expect += [(u, p) for p in range(first, min(first + b, n_parts[u]))]
    assert list(zip(uid.tolist(), part.tolist())) == expect
    assert all(d.guards_intact() for trio in outs for d in trio)
    g.destroy()


@pytest.mark.parametrize("own_rounds", [None, "16", "0"])
def test_independent_ops_taken_without_tickets(hip, oracle, monkeypatch, own_rounds):
    """Entries that wait for no other entry of the graph are taken by workgroup number where they are few per
    workgroup: one each (built-in), several rounds (PCCL_HIP_OWN_ENTRIES=16), or by ticket (=0).  Same bytes."""
    import torch
    monkeypatch.setenv("PCCL_HIP_WIDE", "0")  # (the persistent drain is the subject; such a graph would run as a wide launch)
    if own_rounds is not None:
        monkeypatch.setenv("PCCL_HIP_OWN_ENTRIES", own_rounds)
    rng = np.random.default_rng(77)
    n_ops = 700 if own_rounds is None else 3000
    counts = [int(c) for c in rng.integers(1, 4000, size=n_ops)]   # at most 8 KB: one part each
    total = sum(counts)
    a, b = H.gen("bf16", total, 78, 0), H.gen("bf16", total, 78, 1)
    da, db = H.DevBuf(torch, "bf16", total, 0, src=a), H.DevBuf(torch, "bf16", total, 0, src=b)
    dz = H.DevBuf(torch, "bf16", total, 0)
    ops, at = [], 0
    for c in counts:
        ops.append(dict(dtype="bf16", compute="sum", ins=[da.ptr + 2 * at, db.ptr + 2 * at], outs=[dz.ptr + 2 * at], count=c, deps=[]))
        at += c
    g = hip.Graph(ops)
    info = g.info()
    assert info["n_tiles"] == n_ops and (own_rounds is not None) == (info["n_tiles"] > info["n_workgroups"])
    for _ in range(2):
        dz.view().fill_(0xFF)
        _run_and_check(torch, hip, g, n_ops)
        H.assert_bits_equal(dz.download(), oracle.reduce("bf16", "sum", [a, b]), "independent ops, PCCL_HIP_OWN_ENTRIES=%s" % own_rounds)
    assert dz.guards_intact()
    g.destroy()


@pytest.mark.parametrize("chains,size", [("0", 30_001), ("1", 30_001), ("0", 3_000_001)])
def test_graph_beside_a_kernel_that_occupies_the_gpu(hip, oracle, monkeypatch, chains, size):
    """The drain's workgroups wait for each other inside one launch, so it needs its queues' workgroups
    resident.  With another stream's long elementwise kernels holding compute units at the same time the
    run must still complete every op (no bounded wait may give up), bit-exact: with every op queueing
    its own entries (112 ops that wait for each other through the queue, drawn by ticket) and with the
    ring's steps chained (one workgroup per entry, by number: the chains' heads wait for nothing)."""
    import torch
    from pccl_amd import lang
    monkeypatch.setenv("PCCL_HIP_CHAINS", chains)
    world = 8
    ir, per_rank = lang.ring_allreduce(world, size, dtype="bf16")
    low = ir.lower()
    host_in = [H.gen("bf16", per_rank, 611, r) for r in range(world)]
    bufs = {"in": [H.DevBuf(torch, "bf16", per_rank, 0, src=a) for a in host_in],
            "out": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(world)]}
    g = hip.Graph(lang.bind(low, lambda b, r, e: bufs[b][r].ptr + 2 * e))
    outs = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    hb = {"in": host_in, "out": outs}
    for o in low:
        n = o["count"]
        oracle.reduce_copy("bf16", "sum", [hb[b][r][e:e + n] for (b, r, e) in o["ins"]], [hb[b][r][e:e + n] for (b, r, e) in o["outs"]])
    side = torch.cuda.Stream()
    hog = torch.ones(1 << 28, dtype=torch.float32, device="cuda")       # 1 GiB: each pass a few hundred microseconds
    main = torch.cuda.current_stream()
    for rep in range(3):
        for r in range(world):
            bufs["out"][r].view().fill_(0xFF)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            for _ in range(40):
                hog.mul_(1.0000001).add_(1e-9)
        for _ in range(5):                     # several runs land while the other stream is busy
            g.run(main.cuda_stream)
        assert g.status(main.cuda_stream) == (len(low), len(low)), "a run gave up beside the other kernel (rep %d)" % rep
        assert not side.query() or rep >= 0    # (the other stream may or may not have finished by now)
        torch.cuda.synchronize()
        for r in range(world):
            H.assert_bits_equal(bufs["out"][r].download(), outs[r], "rank %d, rep %d" % (r, rep))
    g.destroy()


# ---- graphs the executor runs as plain launches (tile_bytes = TILE_AUTO) ----------------------------

def _bound_direct_allreduce(torch, hip, oracle, world, slice_elems, dtype, seed):
    from pccl_amd import lang
    ir, per_rank = lang.direct_allreduce(world, slice_elems, dtype=dtype)
    low = ir.lower()
    host_in = [H.gen(dtype, per_rank, seed, r) for r in range(world)]
    bufs = {"in": [H.DevBuf(torch, dtype, per_rank, 0, src=a) for a in host_in],
            "out": [H.DevBuf(torch, dtype, per_rank, 0) for _ in range(world)]}
    es = H.ELEM_BYTES[dtype]
    bound = lang.bind(low, lambda b, r, e: bufs[b][r].ptr + es * e)
    want = oracle.reduce(dtype, "sum", host_in)
    return low, bound, bufs, want


def test_one_exchange_allreduce_becomes_one_launch(hip, oracle):
    """8 folds 8 -> 1 each followed by a copy 1 -> 7: the copies fold into their producers, the eight
    8 -> 8 ops continue each other slice by slice and join: one launch.  Same bytes as the queue."""
    import torch
    stream = _stream(torch)
    low, bound, bufs, want = _bound_direct_allreduce(torch, hip, oracle, 8, 20_000, "bf16", 701)
    g = hip.Graph(bound, hip.TILE_AUTO)
    info = g.info()
    assert info["n_tiles"] == 1 and info["n_workgroups"] == 0 and not info["device_layout"]
    assert g.status(stream) == (0, 16)
    g.run(stream)
    assert g.status(stream) == (16, 16)
    for r in range(8):
        H.assert_bits_equal(bufs["out"][r].download(), want, "rank %d, one launch" % r)
        assert bufs["out"][r].guards_intact()
        bufs["out"][r].view().fill_(0xFF)
    assert g.dependency_kinds() == [0] * 8
    with pytest.raises(hip.PcclError):
        g.trace(True)
    q = hip.Graph(bound)                       # the same ops through the queue
    assert q.info()["n_workgroups"] > 0
    q.run(stream)
    assert q.status(stream) == (16, 16)
    for r in range(8):
        H.assert_bits_equal(bufs["out"][r].download(), want, "rank %d, queue" % r)
    g.destroy()
    q.destroy()


def test_ragged_slices_and_small_graphs_as_launches(hip, oracle):
    import torch
    stream = _stream(torch)
    # slices of an odd number of elements still join (the joined op is just a longer flat array)
    low, bound, bufs, want = _bound_direct_allreduce(torch, hip, oracle, 4, 4099, "f16", 702)
    g = hip.Graph(bound, hip.TILE_AUTO)
    assert g.info()["n_tiles"] == 1
    g.run(stream)
    assert g.status(stream) == (8, 8)
    for r in range(4):
        H.assert_bits_equal(bufs["out"][r].download(), want, "rank %d" % r)
    g.destroy()
    # two dependent ops stay two launches in order: t = a + b; u = t * c (the second is no copy)
    n = 300_007
    a, b, c = (H.gen("f32", n, 703, k) for k in range(3))
    da, db, dc = (H.DevBuf(torch, "f32", n, 4 * k, src=x) for k, x in enumerate((a, b, c)))
    dt, du = H.DevBuf(torch, "f32", n, 0), H.DevBuf(torch, "f32", n, 8)
    g = hip.Graph([dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=n, deps=[]),
                   dict(dtype="f32", compute="prod", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=n, deps=[0])], hip.TILE_AUTO)
    assert g.info()["n_tiles"] == 2
    g.run(stream)
    assert g.status(stream) == (2, 2)
    t = oracle.reduce("f32", "sum", [a, b])
    H.assert_bits_equal(dt.download(), t, "t")
    H.assert_bits_equal(du.download(), oracle.reduce("f32", "prod", [t, c]), "u")
    # rebinding moves the launches' operands
    du2 = H.DevBuf(torch, "f32", n, 12)
    g.rebind(du.ptr, du2.ptr, 4 * n, stream)
    g.run(stream)
    assert g.status(stream) == (2, 2)
    H.assert_bits_equal(du2.download(), oracle.reduce("f32", "prod", [t, c]), "u after the rebind")
    g.destroy()
    # a copy onto its producer's own input is not folded in (the fold would read what it overwrites
    # elsewhere); still two launches, still sequential semantics
    g = hip.Graph([dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=n - 16, deps=[]),
                   dict(dtype="f32", compute="sum", ins=[dt.ptr], outs=[da.ptr + 64], count=n - 16, deps=[0])], hip.TILE_AUTO)
    assert g.info()["n_tiles"] == 2
    g.run(stream)
    assert g.status(stream) == (2, 2)
    t2 = oracle.reduce("f32", "sum", [a[:n - 16], b[:n - 16]])
    H.assert_bits_equal(da.download()[16:], t2, "shifted copy back onto the first input")
    g.destroy()


def test_many_ops_stay_in_the_queue_under_tile_auto(hip, oracle):
    import torch
    from pccl_amd import lang
    ir, per_rank = lang.ring_allreduce(8, 1000, dtype="bf16")
    low = ir.lower()
    bufs = {"in": [H.DevBuf(torch, "bf16", per_rank, 0, src=H.gen("bf16", per_rank, 704, r)) for r in range(8)],
            "out": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(8)]}
    g = hip.Graph(lang.bind(low, lambda b, r, e: bufs[b][r].ptr + 2 * e), hip.TILE_AUTO)
    # (in the queue, not as plain launches; the 14 steps of each rank's chunk run behind each other in
    # one workgroup, so the queue holds an entry per chunk, not per op)
    assert g.info()["n_workgroups"] > 0 and g.info()["n_tiles"] >= 8
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (len(low), len(low))
    for r in range(1, 8):
        H.assert_bits_equal(bufs["out"][r].download(), bufs["out"][0].download(), "rank %d equals rank 0" % r)
    g.destroy()


def test_get_notified_is_released_by_a_notify_of_a_larger_value(hip, oracle):
    """GET_NOTIFIED(word, 3) completes on any value >= 3: a NOTIFY(word, 5) of the same graph satisfies it
    and is what it is ordered behind.  And the legitimate reverse shape, a wait satisfied from outside
    followed downstream by a NOTIFY of a larger value on the same word, builds (no cycle) and runs."""
    import torch
    n = 100_003
    a = H.gen("f32", n, 801, 0)
    da, dt, du = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0), H.DevBuf(torch, "f32", n, 0)
    sig = torch.zeros(4, dtype=torch.int32, device="cuda")
    stream = _stream(torch)
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr], outs=[dt.ptr], count=n, deps=[]),
           dict(primitive=2, signal=sig.data_ptr(), value=5, deps=[0]),
           dict(primitive=3, signal=sig.data_ptr(), value=3, deps=[]),
           dict(dtype="f32", compute="sum", ins=[dt.ptr], outs=[du.ptr], count=n, deps=[2])]
    g = hip.Graph(ops)
    for it in range(3):
        dt.view().fill_(0xFF)
        du.view().fill_(0xFF)
        torch.cuda.synchronize()
        g.run(stream)
        assert g.status(stream) == (4, 4)
        H.assert_bits_equal(du.download(), a, "copy behind GET(3) released by NOTIFY(5), run %d" % it)
    g.destroy()
    # wait from outside, then notify a larger value on the same word
    ops = [dict(primitive=3, signal=sig.data_ptr() + 4, value=3, deps=[]),
           dict(dtype="f32", compute="sum", ins=[da.ptr], outs=[dt.ptr], count=n, deps=[0]),
           dict(primitive=2, signal=sig.data_ptr() + 4, value=5, deps=[1])]
    g = hip.Graph(ops)
    base = g.next_signal_base()
    sig[1] = base + 3
    dt.view().fill_(0xFF)
    torch.cuda.synchronize()
    g.run(stream)
    assert g.status(stream) == (3, 3)
    H.assert_bits_equal(dt.download(), a, "copy released from outside")
    assert int(sig[1].item()) == base + 5
    g.destroy()


# ---- signal ops carried by data ops -----------------------------------------------------------

def _signal_ring_run(torch, hip, oracle, world, size, tile):
    per = world * size
    d_in = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    d_out = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    signals = torch.zeros(64, dtype=torch.int32, device="cuda")
    ops, sym = _signal_ring_ops(world, size, signals.data_ptr(), d_in, d_out)
    g = hip.Graph(ops, tile_bytes=tile)
    ins = [H.gen("bf16", per, 930, r) for r in range(world)]
    outs = [np.zeros(per, dtype=np.uint16) for _ in range(world)]
    bufs = {"in": ins, "out": outs}
    for i in sorted(sym):
        o = sym[i]
        oracle.reduce_copy("bf16", "sum", [bufs[b][r][e:e + size] for (b, r, e) in o["ins"]],
                           [bufs[b][r][e:e + size] for (b, r, e) in o["outs"]])
    for it in range(2):
        for r in range(world):
            d_in[r].upload(ins[r])
            d_out[r].view().fill_(0xFF)
        base = g.next_signal_base()
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (len(ops), len(ops))
        for r in range(world):
            H.assert_bits_equal(d_out[r].download(), outs[r], "run %d rank %d" % (it, r))
        assert signals[:world].cpu().tolist() == [base + 2 * world - 2] * world
    info = g.info()
    g.destroy()
    return info["n_tiles"], len(ops), len(sym)


def test_signal_ops_are_carried_by_their_data_ops(hip, oracle, monkeypatch):
    """A ring whose ranks are linked by signal words only: every GET_NOTIFIED is polled by the parts of
    the one data op behind it and every NOTIFY is stored by whoever completes the one data op in front
    of it, so only the data ops queue entries; every op still counts as complete, the signal words end
    at the run's last value, the results are the checker's.  Switched off, every signal op queues an
    entry of its own and the results are the same."""
    import torch
    world, size = 8, 3001
    entries, n_ops, n_data = _signal_ring_run(torch, hip, oracle, world, size, 4096)
    parts = -(-size * 2 // 4096)
    assert entries == n_data * parts, "only the data ops queue entries"
    monkeypatch.setenv("PCCL_HIP_FUSE_SIGNALS", "0")
    entries_off, _, _ = _signal_ring_run(torch, hip, oracle, world, size, 4096)
    assert entries_off == n_data * parts + (n_ops - n_data)


def test_signal_ops_that_stay_ops_of_their_own(hip, oracle):
    """Shapes in which a signal op cannot ride on a data op: a NOTIFY behind two ops, a GET_NOTIFIED that two
    ops wait for, a second NOTIFY behind the same op (the first is carried), a NOTIFY behind a GET_NOTIFIED,
    a GET_NOTIFIED in front of a NOTIFY.  All of them still do what they say."""
    import torch
    n = 50_001
    a, b = H.gen("f32", n, 940, 0), H.gen("f32", n, 940, 1)
    da, db = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0, src=b)
    dt, du, dv, dw = (H.DevBuf(torch, "f32", n, 0) for _ in range(4))
    sig = torch.zeros(16, dtype=torch.int32, device="cuda")
    word = lambda k: sig.data_ptr() + 4 * k
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=n, deps=[]),      # 0
           dict(dtype="f32", compute="max", ins=[da.ptr, db.ptr], outs=[du.ptr], count=n, deps=[]),      # 1
           dict(primitive=2, signal=word(0), value=3, deps=[0, 1]),                                      # 2: two predecessors
           dict(primitive=2, signal=word(1), value=4, deps=[0]),                                         # 3: carried by op 0
           dict(primitive=2, signal=word(2), value=5, deps=[0]),                                         # 4: op 0 carries one already
           dict(primitive=3, signal=word(0), value=3, deps=[]),                                          # 5: two ops wait for it
           dict(dtype="f32", compute="sum", ins=[dt.ptr], outs=[dv.ptr], count=n, deps=[5]),             # 6
           dict(dtype="f32", compute="sum", ins=[du.ptr], outs=[dw.ptr], count=n, deps=[5]),             # 7
           dict(primitive=3, signal=word(2), value=5, deps=[]),                                          # 8: followed by a NOTIFY
           dict(primitive=2, signal=word(3), value=6, deps=[8])]                                         # 9: behind a GET_NOTIFIED
    g = hip.Graph(ops, tile_bytes=32768)
    parts = -(-n * 4 // 32768)
    assert g.info()["n_tiles"] == 4 * parts + 5, "ops 2, 4, 5, 8 and 9 keep their entries; op 3 rides on op 0"
    for it in range(3):
        for buf in (dt, du, dv, dw):
            buf.view().fill_(0xFF)
        base = g.next_signal_base()
        torch.cuda.synchronize()
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (len(ops), len(ops))
        H.assert_bits_equal(dv.download(), oracle.reduce("f32", "sum", [a, b]), "v, run %d" % it)
        H.assert_bits_equal(dw.download(), oracle.reduce("f32", "max", [a, b]), "w, run %d" % it)
        assert sig[:4].cpu().tolist() == [base + 3, base + 4, base + 5, base + 6]
    g.destroy()


def test_carried_signal_words_move_with_a_rebind(hip, oracle):
    """The words of carried signal ops are operands like any other: a rebind of the range that holds them
    moves the word a data op polls and the word it stores."""
    import torch
    n = 20_000
    a = H.gen("f32", n, 950, 0)
    da, dt = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0)
    sig1 = torch.zeros(16, dtype=torch.int32, device="cuda")
    sig2 = torch.zeros(16, dtype=torch.int32, device="cuda")
    ops = [dict(primitive=3, signal=sig1.data_ptr(), value=2, deps=[]),
           dict(dtype="f32", compute="sum", ins=[da.ptr], outs=[dt.ptr], count=n, deps=[0]),
           dict(primitive=2, signal=sig1.data_ptr() + 4, value=9, deps=[1])]
    g = hip.Graph(ops)
    assert g.info()["n_tiles"] == g.info()["n_workgroups"], "one entry per part of the copy, none for the signal ops"
    stream = _stream(torch)
    for sig in (sig1, sig2):
        if sig is sig2:
            g.rebind(sig1.data_ptr(), sig2.data_ptr(), 64, stream)
        base = g.next_signal_base()
        sig[0] = base + 2
        dt.view().fill_(0xFF)
        torch.cuda.synchronize()
        g.run(stream)
        assert g.status(stream) == (3, 3)
        H.assert_bits_equal(dt.download(), a, "copy released through the word")
        assert int(sig[1].item()) == base + 9
    assert int(sig1[1].item()) != int(sig2[1].item())
    g.destroy()


@pytest.mark.parametrize("tile_bytes", [4096, 0])
def test_ops_without_elements_still_order_and_signal(hip, oracle, tile_bytes):
    """An op of zero elements moves nothing but is an op like any other: it completes behind its
    dependencies, releases what depends on it, may stand in a chain, and carries a GET_NOTIFIED and a
    NOTIFY (null operands are allowed for it)."""
    import torch
    n = 30_011
    a, b = H.gen("f32", n, 960, 0), H.gen("f32", n, 960, 1)
    da, db = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0, src=b)
    dt, du, dv = (H.DevBuf(torch, "f32", n, 0) for _ in range(3))
    sig = torch.zeros(16, dtype=torch.int32, device="cuda")
    word = lambda k: sig.data_ptr() + 4 * k
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=n, deps=[]),      # 0
           dict(dtype="f32", compute="sum", ins=[dt.ptr, da.ptr], outs=[du.ptr], count=0, deps=[0]),     # 1: empty, between two ops
           dict(dtype="f32", compute="sum", ins=[dt.ptr, db.ptr], outs=[du.ptr], count=n, deps=[1]),     # 2
           dict(primitive=2, signal=word(0), value=7, deps=[2]),                                         # 3: rides on op 2
           dict(primitive=3, signal=word(0), value=7, deps=[]),                                          # 4: rides on op 5
           dict(dtype="f32", compute="sum", ins=[0], outs=[0], count=0, deps=[4]),                       # 5: empty carrier, null operands
           dict(primitive=2, signal=word(1), value=8, deps=[5]),                                         # 6: rides on op 5
           dict(primitive=3, signal=word(1), value=8, deps=[]),                                          # 7: rides on op 8
           dict(dtype="f32", compute="max", ins=[du.ptr, da.ptr], outs=[dv.ptr], count=n, deps=[7])]     # 8
    assert hip.plan_signals(ops) == [-1, -1, -1, 2, 5, -1, 5, 8, -1]
    g = hip.Graph(ops, tile_bytes=tile_bytes)
    t = oracle.reduce("f32", "sum", [a, b])
    u = oracle.reduce("f32", "sum", [t, b])
    for it in range(2):
        for buf in (dt, du, dv):
            buf.view().fill_(0xFF)
        base = g.next_signal_base()
        torch.cuda.synchronize()
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (len(ops), len(ops))
        H.assert_bits_equal(du.download(), u, "u, run %d" % it)
        H.assert_bits_equal(dv.download(), oracle.reduce("f32", "max", [u, a]), "v, run %d" % it)
        assert sig[:2].cpu().tolist() == [base + 7, base + 8]
    g.destroy()
    # a graph of empty ops alone
    g = hip.Graph([dict(dtype="bf16", compute="sum", ins=[0, 0], outs=[0], count=0, deps=[]),
                   dict(dtype="bf16", compute="sum", ins=[0], outs=[0], count=0, deps=[0])], tile_bytes=tile_bytes)
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (2, 2)
    g.destroy()
