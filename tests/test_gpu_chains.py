"""GPU parity of chains in the op queue: an op that depends on one op alone, which nothing else
depends on, queues no entries of its own; the workgroup that ran part p of the first goes on with
part p of the second.  Where every later op takes the previous op's output as one of at most two
inputs the whole chain runs in one pass with the value handed on in registers.  Either way the
bits are those of the ops executed one after the other by the CPU checker."""
import numpy as np
import pytest

import helpers as H
import schedules as S

pytestmark = pytest.mark.gpu


def _stream(torch):
    return torch.cuda.current_stream().cuda_stream


class Pool:
    """Named buffers, each on the host (for the CPU checker) and on the device, at a chosen offset
    from a 256-byte boundary."""

    def __init__(self, torch, dtype):
        self.torch, self.dtype, self.host, self.dev = torch, dtype, {}, {}

    def add(self, name, count, offset=0, src=None):
        self.host[name] = np.zeros(count, dtype=H.STORAGE[self.dtype]) if src is None else src.copy()
        self.dev[name] = H.DevBuf(self.torch, self.dtype, count, offset, src=src)
        return self

    def ops_for(self, ops, where):
        out = []
        for o in ops:
            d = dict(o, dtype=self.dtype)
            pick = (lambda n: self.host[n][:o["count"]]) if where == "host" else (lambda n: self.dev[n].ptr)
            d["ins"], d["outs"] = [pick(n) for n in o["ins"]], [pick(n) for n in o["outs"]]
            out.append(d)
        return out

    def check(self, names, what):
        for n in names:
            H.assert_bits_equal(self.dev[n].download(), self.host[n], "%s: %s" % (what, n))
            assert self.dev[n].guards_intact(), "%s: wrote outside %s" % (what, n)


def _run(torch, hip, g, n_ops):
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (n_ops, n_ops)


@pytest.mark.parametrize("dtype,compute", [("bf16", "sum"), ("f16", "max"), ("f32", "sum"), ("f64", "prod"),
                                           ("i32", "min"), ("u32", "max"), ("f8e4m3", "sum"), ("f8e5m2", "max")])
def test_ring_chains_in_one_pass(hip, oracle, monkeypatch, dtype, compute):
    """Ring all-reduce over 8 virtual ranks: per chunk a chain of 14 ops (7 folds, 7 copies).  Chunk
    sizes with elements before the first and behind the last 16-byte pack; operands 16-byte aligned
    or not, inputs and outputs alike in their low address bits or not (down to one element);
    several parts per op or one."""
    import torch
    es = H.ELEM_BYTES[dtype]
    for sizes, offsets, tile in (([1000, 37, 20011], (0, 0), 0), ([5003, 1], (es * 3, es * 3), 0),
                                 ([70001], (es, es), 16 << 10), ([4099], (0, max(4, es)), 8 << 10), ([3001, 50], (es, 3 * es), 0)):
        ops, per_rank = S.ring_allreduce_ops(8, sizes, dtype=dtype, compute=compute)
        # (values near 1 keep a product of eight of them finite)
        kw = dict(mean=1.0, sigma=0.05) if compute == "prod" else dict(sigma=1.0)
        host = {"in": [H.gen(dtype, per_rank, 900, r, **kw) for r in range(8)],
                "out": [np.zeros(per_rank, dtype=H.STORAGE[dtype]) for _ in range(8)]}
        order = oracle.topo_sort(len(ops), S.edges_of(ops))
        oracle.run_ops(S.materialise(ops, lambda b, r, e, n: host[b][r][e:e + n]), order)
        dev = {"in": [H.DevBuf(torch, dtype, per_rank, offsets[0], src=host["in"][r]) for r in range(8)],
               "out": [H.DevBuf(torch, dtype, per_rank, offsets[1]) for _ in range(8)]}
        bound = S.materialise(ops, lambda b, r, e, n: dev[b][r].ptr + e * es)
        monkeypatch.setenv("PCCL_HIP_CHAINS", "0")
        plain = hip.Graph(bound, tile_bytes=tile)
        monkeypatch.setenv("PCCL_HIP_CHAINS", "1")
        # (at most 16 chains and the built-in cut: the graph runs as one launch of chains, a workgroup per 4 KiB;
        # PCCL_HIP_CHAIN_LAUNCH=0: as entries that 14 ops share)
        for chain_launch in ("1", "0"):
            monkeypatch.setenv("PCCL_HIP_CHAIN_LAUNCH", chain_launch)
            g = hip.Graph(bound, tile_bytes=tile)
            if chain_launch == "1" and tile == 0:
                assert g.launch_kind() == "chains", (sizes, offsets)
            if g.launch_kind() != "chains":
                # 14 ops share the entries of one (the built-in choice may also cut a chain into fewer parts)
                if tile:
                    assert g.info()["n_tiles"] * 14 == plain.info()["n_tiles"], (sizes, offsets)
                else:
                    assert g.info()["n_tiles"] * 14 <= plain.info()["n_tiles"], (sizes, offsets)
            for it in range(2):
                for b in dev["out"]:
                    b.view().fill_(0xFF)
                _run(torch, hip, g, len(ops))
                for r in range(8):
                    H.assert_bits_equal(dev["out"][r].download(), host["out"][r], "%s %s sizes %s offsets %s run %d rank %d (%s)"
                                        % (dtype, compute, sizes, offsets, it, r, g.launch_kind()))
                    assert dev["out"][r].guards_intact()
            g.destroy()
        plain.destroy()
        monkeypatch.delenv("PCCL_HIP_CHAIN_LAUNCH")


def test_two_outputs_and_value_handed_on_as_second_input(hip, oracle):
    """t, t2 = a + b;  u = c + t (the handed-on value is input 1);  v, w = copy(u);  x = v + d."""
    import torch
    for count, offset in ((100003, 0), (9, 8), (3 * 1000 * 1000 + 5, 4)):
        pool = Pool(torch, "f32")
        for k, n in enumerate("abcd"):
            pool.add(n, count, offset, src=H.gen("f32", count, 910, k))
        for n in ("t", "t2", "u", "v", "w", "x"):
            pool.add(n, count, offset)
        ops = [dict(compute="sum", ins=["a", "b"], outs=["t", "t2"], count=count, deps=[]),
               dict(compute="sum", ins=["c", "t"], outs=["u"], count=count, deps=[0]),
               dict(compute="sum", ins=["u"], outs=["v", "w"], count=count, deps=[1]),
               dict(compute="sum", ins=["v", "d"], outs=["x"], count=count, deps=[2])]
        oracle.run_ops(pool.ops_for(ops, "host"))
        g = hip.Graph(pool.ops_for(ops, "dev"))
        assert g.info()["n_tiles"] >= 1
        _run(torch, hip, g, 4)
        pool.check(("t", "t2", "u", "v", "w", "x"), "count %d offset %d" % (count, offset))
        g.destroy()


def test_chain_that_reads_what_it_wrote_earlier_goes_through_memory(hip, oracle):
    """t = a + b;  u = t + c;  t = u + t (in place, reads op 0's output again);  v = copy(t): the ops still
    run behind each other in one workgroup, but every op reads its inputs from memory."""
    import torch
    for count in (200003, 5 * 1000 * 1000 + 1):
        pool = Pool(torch, "bf16")
        for k, n in enumerate("abc"):
            pool.add(n, count, 0, src=H.gen("bf16", count, 920, k))
        for n in "tuv":
            pool.add(n, count, 0)
        ops = [dict(compute="sum", ins=["a", "b"], outs=["t"], count=count, deps=[]),
               dict(compute="sum", ins=["t", "c"], outs=["u"], count=count, deps=[0]),
               dict(compute="sum", ins=["u", "t"], outs=["t"], count=count, deps=[1]),
               dict(compute="sum", ins=["t"], outs=["v"], count=count, deps=[2])]
        oracle.run_ops(pool.ops_for(ops, "host"))
        g = hip.Graph(pool.ops_for(ops, "dev"))
        _run(torch, hip, g, 4)
        pool.check("tuv", "count %d" % count)
        g.destroy()


@pytest.mark.parametrize("fold", ["1", "0"])
def test_copy_of_the_previous_ops_output_is_stored_by_that_op(hip, oracle, monkeypatch, fold):
    """t = fold of 3..8 inputs;  v0..v6 = copy(t);  w = copy(v0);  x = copy(w): the chain goes through memory (more than
    two inputs), the first copy's outputs are stored by the fold itself, the second copy runs by itself, the third
    is stored by the second.  Ragged counts, operands off the 16-byte grid, one part and several;
    PCCL_HIP_FOLD_COPIES=0 runs every op by itself.  Same bytes either way."""
    import torch
    monkeypatch.setenv("PCCL_HIP_FOLD_COPIES", fold)
    for dtype, compute, n_in, n_copy, count, offset, tile in (("bf16", "sum", 8, 7, 300_007, 0, 0), ("f32", "max", 3, 5, 70_001, 4, 16 << 10),
                                                              ("f16", "prod", 5, 3, 1_000_003, 6, 64 << 10), ("i32", "sum", 8, 7, 4_099, 12, 0),
                                                              ("f8e5m2", "sum", 4, 4, 250_001, 3, 0), ("f64", "min", 6, 2, 65_537, 8, 0)):
        pool = Pool(torch, dtype)
        names_in = ["in%d" % k for k in range(n_in)]
        for k, n in enumerate(names_in):
            src = H.gen(dtype, count, 930, k, kind="uniform", lo=0.5, hi=2.0) if compute == "prod" else H.gen(dtype, count, 930, k)
            pool.add(n, count, offset if k % 2 else 0, src=src)
        copies = ["v%d" % k for k in range(n_copy)]
        for k, n in enumerate(["t"] + copies + ["w", "x"]):
            pool.add(n, count, (offset * (k % 3)) % 64)
        ops = [dict(compute=compute, ins=names_in, outs=["t"], count=count, deps=[]),
               dict(compute=compute, ins=["t"], outs=copies, count=count, deps=[0]),
               dict(compute=compute, ins=["v0"], outs=["w"], count=count, deps=[1]),
               dict(compute=compute, ins=["w"], outs=["x"], count=count, deps=[2])]
        oracle.run_ops(pool.ops_for(ops, "host"))
        bound = pool.ops_for(ops, "dev")
        plan = hip.plan_chains(bound, [1] * 4, H.ELEM_BYTES[dtype])
        assert [p[2] for p in plan] == ([0, 2, 0, 2] if fold == "1" else [0, 0, 0, 0])
        g = hip.Graph(bound, tile_bytes=tile)
        for run in range(2):
            for n in ["t", "w", "x"] + copies:
                pool.dev[n].view().fill_(0xFF)
            _run(torch, hip, g, 4)
            pool.check(["t", "w", "x"] + copies, "%s %s %d -> 1 -> %d, count %d, run %d" % (dtype, compute, n_in, n_copy, count, run))
        g.destroy()


def test_mixed_computes_and_more_ops_than_one_pass_holds(hip, oracle):
    """x1 = x0 + a, x2 = max(x1, b), x3 = x2 * c, ... 20 ops in a row: ops that do not share one
    fold run in the kernel instance that picks the fold per op, which takes chains through memory;
    the same 20 ops with one fold are more than one pass holds and go through memory as well."""
    import torch
    count = 50021
    for computes in (["sum", "max", "prod", "min"] * 5, ["sum"] * 20):
        pool = Pool(torch, "f32")
        for k, n in enumerate("abc"):
            pool.add(n, count, 0, src=H.gen("f32", count, 930, k, mean=1.0, sigma=0.1))
        for k in range(21):
            pool.add("x%d" % k, count, 0, src=H.gen("f32", count, 930, 5) if k == 0 else None)
        ops = [dict(compute=c, ins=["x%d" % k, "abc"[k % 3]], outs=["x%d" % (k + 1)], count=count, deps=[k - 1] if k else [])
               for k, c in enumerate(computes)]
        oracle.run_ops(pool.ops_for(ops, "host"))
        g = hip.Graph(pool.ops_for(ops, "dev"), tile_bytes=64 << 10)
        assert g.info()["n_tiles"] == 4  # one chain, four parts
        _run(torch, hip, g, 20)
        pool.check(["x%d" % k for k in range(1, 21)], "computes %s" % computes[:4])
        g.destroy()


def test_chains_between_a_fan_out_and_a_fan_in(hip, oracle):
    """s = a + b feeds two chains of four ops each; z = (end of chain 1) + (end of chain 2).  The head of a
    chain waits for s, and z waits for both chains' last ops."""
    import torch
    for count, tile in ((1000, 0), (700001, 16 << 10)):
        pool = Pool(torch, "bf16")
        for k, n in enumerate("abcd"):
            pool.add(n, count, 0, src=H.gen("bf16", count, 940, k))
        names = ["s", "z"] + ["p%d" % k for k in range(4)] + ["q%d" % k for k in range(4)]
        for n in names:
            pool.add(n, count, 0)
        ops = [dict(compute="sum", ins=["a", "b"], outs=["s"], count=count, deps=[])]
        for chain, extra in (("p", "c"), ("q", "d")):
            for k in range(4):
                src = "s" if k == 0 else "%s%d" % (chain, k - 1)
                dep = 0 if k == 0 else len(ops) - 1
                ops.append(dict(compute="sum", ins=[src, extra] if k % 2 == 0 else [src], outs=["%s%d" % (chain, k)],
                                count=count, deps=[dep]))
        ops.append(dict(compute="sum", ins=["p3", "q3"], outs=["z"], count=count, deps=[4, 8]))
        oracle.run_ops(pool.ops_for(ops, "host"))
        g = hip.Graph(pool.ops_for(ops, "dev"), tile_bytes=tile)
        for _ in range(3):  # the graph re-arms itself
            for n in names:
                pool.dev[n].view().fill_(0xFF)
            _run(torch, hip, g, len(ops))
            pool.check(names, "count %d" % count)
        g.destroy()


def test_rebind_moves_the_chains_operands(hip, oracle):
    """A chain that runs in one pass keeps its operand addresses in a table beside the payloads;
    graph_rebind moves both, to a buffer of the same alignment and to one 4 bytes off it."""
    import torch
    count = 300007
    pool = Pool(torch, "f32")
    for k, n in enumerate("abc"):
        pool.add(n, count, 0, src=H.gen("f32", count, 950, k))
    for n in ("t", "u", "v"):
        pool.add(n, count, 0)
    ops = [dict(compute="sum", ins=["a", "b"], outs=["t"], count=count, deps=[]),
           dict(compute="sum", ins=["t", "c"], outs=["u"], count=count, deps=[0]),
           dict(compute="sum", ins=["u"], outs=["v"], count=count, deps=[1])]
    oracle.run_ops(pool.ops_for(ops, "host"))
    g = hip.Graph(pool.ops_for(ops, "dev"))
    entries = g.info()["n_tiles"]
    _run(torch, hip, g, 3)
    pool.check("tuv", "before the rebind")
    # u moves to a fresh buffer with the same alignment, then to one 4 bytes off it
    at = pool.dev["u"]
    for offset in (0, 4):
        moved = H.DevBuf(torch, "f32", count, offset)
        g.rebind(at.ptr, moved.ptr, 4 * count, _stream(torch))
        assert g.info()["n_tiles"] == entries
        at.view().fill_(0x11)
        pool.dev["v"].view().fill_(0xFF)
        _run(torch, hip, g, 3)
        H.assert_bits_equal(moved.download(), pool.host["u"], "u after the move (offset %d)" % offset)
        assert moved.guards_intact()
        pool.check("tv", "after the move (offset %d)" % offset)
        assert (at.download().view(np.uint32) == 0x11111111).all(), "the old buffer was written after the rebind"
        keep = at  # (alive until the next rebind has gone through)
        at = moved
    g.destroy()


def test_chains_of_copies_with_an_element_size_of_their_own(hip, oracle):
    """A copy moves bytes of its own dtype, whatever the graph's REDUCE ops are: chains of copies in a
    graph without any REDUCE op (the kernel instance then follows the first op's dtype), and chains of
    f64 / f32 / 1-byte copies beside bf16 reductions."""
    import torch
    count = 70003
    for reduce_dtype, copy_dtypes in ((None, ["f64", "f32", "f8e4m3"]), (None, ["bf16", "f64"]), ("bf16", ["f64", "f32", "f8e5m2", "bf16"])):
        ops_dev, ops_host, checks, sources = [], [], [], []
        if reduce_dtype:
            a, b = H.gen(reduce_dtype, count, 960, 0), H.gen(reduce_dtype, count, 960, 1)
            da, db = H.DevBuf(torch, reduce_dtype, count, 0, src=a), H.DevBuf(torch, reduce_dtype, count, 0, src=b)
            dt = H.DevBuf(torch, reduce_dtype, count, 0)
            ht = np.zeros(count, dtype=H.STORAGE[reduce_dtype])
            ops_dev.append(dict(dtype=reduce_dtype, compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]))
            ops_host.append(dict(dtype=reduce_dtype, compute="sum", ins=[a, b], outs=[ht], count=count))
            checks.append((dt, ht, "sum"))
        for k, dtype in enumerate(copy_dtypes):
            src = H.gen(dtype, count, 961, k)
            dev = [H.DevBuf(torch, dtype, count, H.ELEM_BYTES[dtype] * (j % 3), src=src if j == 0 else None) for j in range(5)]
            sources.append(dev[0])  # (stays allocated while the graph reads it)
            host = [src] + [np.zeros(count, dtype=H.STORAGE[dtype]) for _ in range(4)]
            for j in range(4):  # x0 -> x1 -> x2 -> x3 -> x4
                deps = [len(ops_dev) - 1] if j else []
                ops_dev.append(dict(dtype=dtype, compute="sum", ins=[dev[j].ptr], outs=[dev[j + 1].ptr], count=count, deps=deps))
                ops_host.append(dict(dtype=dtype, compute="sum", ins=[host[j]], outs=[host[j + 1]], count=count))
                checks.append((dev[j + 1], host[j + 1], "%s copy %d" % (dtype, j)))
        oracle.run_ops(ops_host)
        for tile in (1 << 20, 16 << 10):
            g = hip.Graph(ops_dev, tile_bytes=tile)
            if tile == 1 << 20:  # one part per op: an entry per chain of copies, one for the reduction
                assert g.info()["n_tiles"] == len(copy_dtypes) + (1 if reduce_dtype else 0)
            for dev_buf, _, _ in checks:
                dev_buf.view().fill_(0xFF)
            _run(torch, hip, g, len(ops_dev))
            for dev_buf, want, what in checks:
                H.assert_bits_equal(dev_buf.download(), want, "%s (reduce dtype %s, parts of %d)" % (what, reduce_dtype, tile))
                assert dev_buf.guards_intact(), what
            g.destroy()


def test_an_output_written_again_later_in_the_chain(hip, oracle):
    """t, keep = a + b;  t = t + c (in place);  u = copy(t);  t = u + d (writes t a third time);  w = t + a: one
    chain, run in one pass, which may skip the stores of t that it overwrites itself.  x = copy(t) and
    y = t + keep run behind it and read what the chain left in memory, which must be what the ops leave
    when run one by one."""
    import torch
    for count, tile in ((50021, 0), (9, 0), (2 * 1000 * 1000 + 3, 32 << 10)):
        pool = Pool(torch, "bf16")
        for k, n in enumerate("abcd"):
            pool.add(n, count, 0, src=H.gen("bf16", count, 970, k))
        names = ("t", "keep", "u", "w", "x", "y")
        for n in names:
            pool.add(n, count, 0)
        ops = [dict(compute="sum", ins=["a", "b"], outs=["t", "keep"], count=count, deps=[]),
               dict(compute="sum", ins=["t", "c"], outs=["t"], count=count, deps=[0]),
               dict(compute="sum", ins=["t"], outs=["u"], count=count, deps=[1]),
               dict(compute="sum", ins=["u", "d"], outs=["t"], count=count, deps=[2]),
               dict(compute="sum", ins=["t", "a"], outs=["w"], count=count, deps=[3]),
               dict(compute="sum", ins=["t"], outs=["x"], count=count, deps=[4]),
               dict(compute="sum", ins=["t", "keep"], outs=["y"], count=count, deps=[4])]
        oracle.run_ops(pool.ops_for(ops, "host"))
        plan = hip.plan_chains(pool.ops_for(ops, "dev"), [1] * 7, 2)
        assert [p[0] for p in plan] == [1, 2, 3, 4, -1, -1, -1] and plan[0][1:3] == (5, 1)  # one chain of 5, one pass
        g = hip.Graph(pool.ops_for(ops, "dev"), tile_bytes=tile)
        for _ in range(2):
            for n in names:
                pool.dev[n].view().fill_(0xFF)
            _run(torch, hip, g, 7)
            pool.check(names, "count %d" % count)
        g.destroy()


def _random_chain_graph(rng, torch, dtype, compute, count):
    """Several chains in one graph.  Each chain: a first op with one or two inputs, then 1..19 ops that
    mostly take the previous op's output 0 (as input 0 or 1, alone or with an outside buffer), sometimes
    read an earlier output of the chain instead of an outside buffer, write one or two outputs, and
    sometimes write over an earlier output of the chain or work in place.  Returns named buffers
    (host + device) and the ops in both forms."""
    es = H.ELEM_BYTES[dtype]
    host, dev = {}, {}

    def new(name, src=None):
        off = int(rng.integers(0, 4)) * es if rng.random() < 0.5 else 0
        host[name] = np.zeros(count, dtype=H.STORAGE[dtype]) if src is None else src
        dev[name] = H.DevBuf(torch, dtype, count, off, src=src)
        return name

    kw = dict(kind="uniform", lo=0.5, hi=1.5) if compute == "prod" and dtype not in ("i32", "u32") else {}
    if compute == "prod" and dtype in ("i32", "u32"):
        kw = dict(lo=0, hi=3)
    outside = [new("in%d" % k, H.gen(dtype, count, int(rng.integers(1 << 20)), k, **kw)) for k in range(4)]
    ops = []
    for c in range(int(rng.integers(1, 4))):
        written = []  # buffers this chain has written (no other chain touches them; `outside` is read-only)
        for s in range(int(rng.integers(2, 21))):
            if s == 0:
                ins = [outside[k] for k in rng.permutation(4)[:int(rng.integers(1, 3))]]
            else:
                handed = ops[-1]["outs"][0]
                earlier = [n for n in written if n != handed]
                r = rng.random()
                if r < 0.35:
                    ins = [handed]
                elif r < 0.9 or not earlier:
                    ins = [handed, outside[int(rng.integers(4))]]
                else:  # reads something else the chain wrote earlier: such a chain goes through memory
                    ins = [handed, earlier[int(rng.integers(len(earlier)))]]
                if len(ins) == 2 and rng.random() < 0.5:
                    ins.reverse()
            outs = []
            for j in range(1 if rng.random() < 0.75 else 2):
                r = rng.random()
                again = [n for n in written if n not in outs]
                if r < 0.2 and again:
                    outs.append(again[int(rng.integers(len(again)))])   # writes an earlier output again (maybe in place)
                else:
                    outs.append(new("c%d_%d_%d" % (c, s, j)))
            ops.append(dict(compute=compute, ins=ins, outs=outs, count=count, deps=[len(ops) - 1] if s else []))
            written += [n for n in outs if n not in written]
    return host, dev, ops


def test_random_chains(hip, oracle):
    """Seeded sweep over chains of 2..20 ops with one or two inputs and outputs per op, operands at
    arbitrary element-aligned offsets, ops that work in place, write over or read again what the chain
    wrote earlier, all dtypes and folds, one part per op and several: bit for bit the memory that the
    ops leave when run one after the other."""
    import torch
    scale = max(1, int(__import__("os").environ.get("PCCL_TEST_SWEEP_SCALE", "1")))
    rng = np.random.default_rng(20240 + (0 if scale == 1 else 7919))
    dtypes = ["f32", "i32", "bf16", "f16", "f8e4m3", "f8e5m2", "f64", "u32"]
    one_pass = 0
    for case in range(60 * scale):
        dtype = dtypes[int(rng.integers(len(dtypes)))]
        compute = ["sum", "prod", "min", "max"][int(rng.integers(4))]
        count = int(np.exp(rng.uniform(0, np.log(200_000))))
        host, dev, ops = _random_chain_graph(rng, torch, dtype, compute, count)
        bound = lambda where: [dict(o, dtype=dtype, ins=[(host[n] if where == "host" else dev[n].ptr) for n in o["ins"]],
                                    outs=[(host[n] if where == "host" else dev[n].ptr) for n in o["outs"]]) for o in ops]
        oracle.run_ops(bound("host"))
        tile = [0, 4096, 16 << 10, 1 << 20][int(rng.integers(4))]
        plan = hip.plan_chains(bound("dev"), [1] * len(ops), H.ELEM_BYTES[dtype])
        one_pass += sum(1 for p in plan if p[0] >= 0 and p[1] > 1 and p[2] == 1)
        g = hip.Graph(bound("dev"), tile_bytes=tile)
        for run in range(2):
            _run(torch, hip, g, len(ops))
            if run == 0:  # the second run starts from what the first left (in-place ops): compare after the first,
                what = "case %d (%s %s count %d, %d ops, parts of %d)" % (case, dtype, compute, count, len(ops), tile)
                for n in host:
                    got, want = dev[n].download(), host[n]
                    if dtype in ("f8e4m3", "f8e5m2"):  # any NaN encoding of the format counts as NaN
                        wn, gn = np.isnan(oracle.widen(dtype, want)), np.isnan(oracle.widen(dtype, got))
                        assert np.array_equal(wn, gn), what + ": NaN positions in " + n
                        got, want = np.where(wn, 0, got), np.where(wn, 0, want)
                    H.assert_bits_equal(got, want, what + ": " + n)
                    assert dev[n].guards_intact(), what + ": wrote outside " + n
                break
        g.destroy()
    assert one_pass >= 20 * scale  # the sweep does reach the one-pass code


def test_later_op_writes_over_an_earlier_output_at_a_shift(hip, oracle):
    """t = a + b;  u = t + c;  t[16:] = copy(u): the last op's output overlaps the first op's 16 elements
    further on.  Different lanes would write those elements in a one-pass chain, so the chain goes
    through memory, where the later op's values are the ones that stay."""
    import torch
    for count in (1000, 300007):
        a, b, c = (H.gen("f32", count, 980, k) for k in range(3))
        da, db, dc = (H.DevBuf(torch, "f32", count, 0, src=x) for x in (a, b, c))
        dt, du = H.DevBuf(torch, "f32", count + 16, 0), H.DevBuf(torch, "f32", count, 0)
        ht, hu = np.zeros(count + 16, dtype=np.float32), np.zeros(count, dtype=np.float32)
        ht.view(np.uint32)[:] = 0xFFFFFFFF
        host_ops = [dict(dtype="f32", compute="sum", ins=[a, b], outs=[ht[:count]], count=count),
                    dict(dtype="f32", compute="sum", ins=[ht[:count], c], outs=[hu], count=count),
                    dict(dtype="f32", compute="sum", ins=[hu], outs=[ht[16:]], count=count)]
        oracle.run_ops(host_ops)
        ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
               dict(dtype="f32", compute="sum", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[0]),
               dict(dtype="f32", compute="sum", ins=[du.ptr], outs=[dt.ptr + 64], count=count, deps=[1])]
        plan = hip.plan_chains(ops, [1, 1, 1], 4)
        assert [p[0] for p in plan] == [1, 2, -1] and plan[0][2] == 0   # one chain, not in one pass
        g = hip.Graph(ops, tile_bytes=1 << 22)   # one part per op (several parts: the last dependency waits for the whole op)
        for _ in range(3):
            dt.view().fill_(0xFF)
            _run(torch, hip, g, 3)
            H.assert_bits_equal(dt.download(), ht, "t, count %d" % count)
            H.assert_bits_equal(du.download(), hu, "u, count %d" % count)
        g.destroy()
        g = hip.Graph(ops, tile_bytes=16 << 10)
        dt.view().fill_(0xFF)
        _run(torch, hip, g, 3)
        H.assert_bits_equal(dt.download(), ht, "t, count %d, several parts" % count)
        g.destroy()


@pytest.mark.parametrize("dtype,compute", [("bf16", "sum"), ("f32", "prod"), ("f64", "min"), ("f8e4m3", "max"), ("i32", "sum")])
def test_folds_and_their_broadcast_copies_as_one_launch_of_chains(hip, oracle, monkeypatch, dtype, compute):
    """A direct all-reduce over 8 ranks (rank r folds slice r of all inputs, a copy broadcasts the result:
    16 ops, 8 queue entries), none of whose entries waits for anything: the graph runs as one launch of
    chains, a workgroup per 4 KiB, whatever the operands' alignment.  With independent ops of 1..8 inputs and
    several outputs beside it (copies and thin folds, for which that launch is not the library's choice:
    PCCL_HIP_CHAIN_LAUNCH=2 takes it wherever the graph fits): bits as from the table-driven wide launch,
    through the persistent drain, and as the CPU checker's."""
    import torch
    es = H.ELEM_BYTES[dtype]
    kw = dict(mean=1.0, sigma=0.05) if compute == "prod" else dict(sigma=1.0)
    for slice_elems, offsets in ((4096 // es * 3, (0, 0)), (1237, (es, 3 * es)), (7, (es, 0)), (40001, (0, max(4, es)))):
        per_rank = 8 * slice_elems
        host_in = [H.gen(dtype, per_rank, 1200, r, **kw) for r in range(8)]
        dev_in = [H.DevBuf(torch, dtype, per_rank, offsets[0], src=host_in[r]) for r in range(8)]
        dev_out = [H.DevBuf(torch, dtype, per_rank, offsets[1]) for _ in range(8)]
        ops, want = [], [np.zeros(per_rank, dtype=H.STORAGE[dtype]) for _ in range(8)]
        for r in range(8):
            lo = r * slice_elems
            ops.append(dict(dtype=dtype, compute=compute, ins=[d.ptr + lo * es for d in dev_in], outs=[dev_out[r].ptr + lo * es],
                            count=slice_elems, deps=[]))
            ops.append(dict(dtype=dtype, compute=compute, ins=[dev_out[r].ptr + lo * es],
                            outs=[dev_out[d].ptr + lo * es for d in range(8) if d != r], count=slice_elems, deps=[len(ops) - 1]))
            folded = oracle.reduce(dtype, compute, [x[lo:lo + slice_elems] for x in host_in])
            for d in range(8):
                want[d][lo:lo + slice_elems] = folded
        g = hip.Graph(ops)
        assert g.launch_kind() == "chains", (g.launch_kind(), slice_elems)  # (the library's own choice for these folds)
        g.destroy()
        extra = []
        for k, (n_in, n_out, count) in enumerate(((1, 3, 5000), (3, 2, 999), (8, 1, 12345), (2, 8, 1), (5, 1, 4096 // es), (1, 1, 70001))):
            srcs = [H.gen(dtype, count, 1300 + k, j, **kw) for j in range(n_in)]
            ds = [H.DevBuf(torch, dtype, count, ((k + j) % 5) * es, src=x) for j, x in enumerate(srcs)]
            do = [H.DevBuf(torch, dtype, count, ((k + 2 * j) % 7) * es) for j in range(n_out)]
            ops.append(dict(dtype=dtype, compute=compute, ins=[d.ptr for d in ds], outs=[d.ptr for d in do], count=count, deps=[]))
            extra.append((do, oracle.reduce(dtype, compute, srcs) if n_in > 1 else srcs[0], ds))
        for form, env in (("chains", {"PCCL_HIP_CHAIN_LAUNCH": "2"}), ("wide", {}), ("wide", {"PCCL_HIP_CHAIN_LAUNCH": "0"}), ("drain", {"PCCL_HIP_WIDE": "0"})):
            for k, v in env.items():
                monkeypatch.setenv(k, v)
            g = hip.Graph(ops)
            for k in env:
                monkeypatch.delenv(k)
            assert g.launch_kind() == form, (form, g.launch_kind(), slice_elems)
            if form == "chains":
                g.trace(True)
            for it in range(2):
                for b in dev_out + [b for do, _, _ in extra for b in do]:
                    b.view().fill_(0xFF)
                _run(torch, hip, g, len(ops))
                for r in range(8):
                    H.assert_bits_equal(dev_out[r].download(), want[r], "%s %s %s slice %d run %d rank %d" % (form, dtype, compute, slice_elems, it, r))
                    assert dev_out[r].guards_intact()
                for k, (do, w, _) in enumerate(extra):
                    for b in do:
                        H.assert_bits_equal(b.download(), w, "%s %s %s extra op %d" % (form, dtype, compute, k))
                        assert b.guards_intact()
            if form == "chains":
                tr = g.read_trace(_stream(torch))
                info = g.info()
                assert len(tr) == info["n_workgroups"] == info["n_tiles"] and (tr[:, 3] >= tr[:, 1]).all() and (tr[:, 1] > 0).all()
            g.destroy()


def test_launch_of_chains_follows_rebinds_also_when_recorded(hip, oracle):
    """A ring all-reduce over 8 ranks that runs as one launch of chains: its operands move to other tensors
    (other alignment included) by rebinds, eagerly and between replays of a HIP graph that recorded the
    launch: the table of the chains' operands lives in the graph's arena, so the recorded launch follows.
    A rebind that changes the chains themselves (the output tensor becomes the input tensor) is refused
    and leaves the graph as it was."""
    import torch
    dtype, es = "bf16", 2
    ops, per_rank = S.ring_allreduce_ops(8, [3001], dtype=dtype, compute="sum")
    host = {"in": [H.gen(dtype, per_rank, 1400, r) for r in range(8)], "out": [np.zeros(per_rank, dtype=H.STORAGE[dtype]) for _ in range(8)]}
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: host[b][r][e:e + n]), oracle.topo_sort(len(ops), S.edges_of(ops)))
    # all ranks' tensors in one allocation each, so that one rebind moves all eight
    ins = H.DevBuf(torch, dtype, 8 * per_rank, 0, src=np.concatenate(host["in"]))
    outs = [H.DevBuf(torch, dtype, 8 * per_rank, off) for off in (0, 4, 40)]
    ins2 = H.DevBuf(torch, dtype, 8 * per_rank, 12, src=np.concatenate(host["in"]))
    where = {"in": ins, "out": outs[0]}
    g = hip.Graph(S.materialise(ops, lambda b, r, e, n: where[b].ptr + (r * per_rank + e) * es))
    assert g.launch_kind() == "chains"
    stream = torch.cuda.Stream()
    want = np.concatenate(host["out"])

    def check(buf, what):
        H.assert_bits_equal(buf.download(), want, what)
        assert buf.guards_intact()

    with torch.cuda.stream(stream):
        g.run(stream.cuda_stream)
        stream.synchronize()
        check(outs[0], "eager")
        g.rebind(outs[0].ptr, outs[1].ptr, 8 * per_rank * es, stream.cuda_stream)
        g.rebind(ins.ptr, ins2.ptr, 8 * per_rank * es, stream.cuda_stream)
        g.run(stream.cuda_stream)
        stream.synchronize()
        check(outs[1], "after rebinds to tensors of another alignment")
        with pytest.raises(hip.PcclError) as e:
            g.rebind(outs[1].ptr, ins2.ptr, 8 * per_rank * es, stream.cuda_stream)
        assert e.value.code == hip.ERR_UNSUPPORTED
        cg = torch.cuda.CUDAGraph()
        with torch.cuda.graph(cg, stream=stream):
            g.run(stream.cuda_stream)
        current = outs[1]
        for target in (outs[2], outs[0], outs[1]):
            g.rebind(current.ptr, target.ptr, 8 * per_rank * es, stream.cuda_stream)
            current = target
            target.view().fill_(0xFF)
            stream.synchronize()
            cg.replay()
            stream.synchronize()
            check(target, "replay after a rebind")
    assert g.status(stream.cuda_stream) == (len(ops), len(ops))
    g.destroy()


@pytest.mark.parametrize("collective", ["ring_reduce_scatter", "ring_all_gather", "all_to_all", "broadcast"])
def test_other_collectives_over_resident_ranks_in_every_form(hip, oracle, monkeypatch, collective):
    """The other collectives of the schedule language over 8 ranks that live on this device.  All-gather (chains
    of copies), all-to-all (64 independent copies) and broadcast (one copy to seven outputs) fit the launch of
    chains but are better off as the table-driven wide launch, which is the library's choice;
    PCCL_HIP_CHAIN_LAUNCH=2 takes the launch of chains for them.  A ring reduce-scatter's chains leave their
    partial sums in memory, which that launch cannot do: wide either way.  Same bits in every form."""
    import torch
    from pccl_amd import lang
    dtype, es, chunk = "bf16", 2, 2501
    emit = getattr(lang, collective)
    ir, per_rank = emit(8, chunk, dtype=dtype) if collective != "broadcast" else emit(8, 8 * chunk, dtype=dtype)
    low = ir.lower()
    host = {"in": [H.gen(dtype, per_rank, 1500, r) for r in range(8)], "out": [np.zeros(per_rank, dtype=H.STORAGE[dtype]) for _ in range(8)]}
    dev = {"in": [H.DevBuf(torch, dtype, per_rank, 2 * (r % 3), src=host["in"][r]) for r in range(8)],
           "out": [H.DevBuf(torch, dtype, per_rank, 2 * (r % 5)) for r in range(8)]}
    h_ops = lang.bind(low, lambda b, r, e: host[b][r][e:])
    for o in h_ops:  # (the CPU checker takes arrays of the op's length)
        o["ins"], o["outs"] = [x[:o["count"]] for x in o["ins"]], [x[:o["count"]] for x in o["outs"]]
    oracle.run_ops(h_ops, oracle.topo_sort(len(h_ops), [(d, i) for i, o in enumerate(h_ops) for d in o.get("deps", [])]))
    forced = "wide" if collective == "ring_reduce_scatter" else "chains"
    for want, env in ((forced, {"PCCL_HIP_CHAIN_LAUNCH": "2"}), ("wide", {}), ("drain", {"PCCL_HIP_WIDE": "0"})):
        for k, v in env.items():
            monkeypatch.setenv(k, v)
        g = hip.Graph(lang.bind(low, lambda b, r, e: dev[b][r].ptr + e * es))
        for k in env:
            monkeypatch.delenv(k)
        assert g.launch_kind() == want, (want, g.launch_kind())
        for it in range(2):
            for b in dev["out"]:
                b.upload(np.zeros(per_rank, dtype=H.STORAGE[dtype]))
            _run(torch, hip, g, len(low))
            for r in range(8):
                H.assert_bits_equal(dev["out"][r].download(), host["out"][r], "%s as %s run %d rank %d" % (collective, want, it, r))
                assert dev["out"][r].guards_intact()
        g.destroy()


def test_large_fan_out_copies_run_as_a_launch_of_chains(hip, oracle):
    """An all-gather over 8 resident ranks whose chains of copies move 72 MiB in all: from 48 MiB such a graph
    runs as a launch of chains with non-temporal stores (what a direct launch gives a copy to many outputs).
    Every rank's output is the concatenation of the ranks' chunks."""
    import torch
    from pccl_amd import lang
    chunk = (1 << 19) + 24  # elements per chunk: 1 MiB and a few packs
    ir, per_rank = lang.ring_all_gather(8, chunk, dtype="bf16")
    low = ir.lower()
    src = [H.gen("bf16", per_rank, 1600, r) for r in range(8)]
    dev = {"in": [H.DevBuf(torch, "bf16", per_rank, 0, src=src[r]) for r in range(8)],
           "out": [H.DevBuf(torch, "bf16", per_rank, 16 * (r % 2)) for r in range(8)]}
    g = hip.Graph(lang.bind(low, lambda b, r, e: dev[b][r].ptr + 2 * e))
    assert g.launch_kind() == "chains", g.launch_kind()
    want = np.concatenate([src[r][r * chunk:(r + 1) * chunk] for r in range(8)])
    for it in range(2):
        for b in dev["out"]:
            b.view().fill_(0xFF)
        _run(torch, hip, g, len(low))
        for r in range(8):
            H.assert_bits_equal(dev["out"][r].download(), want, "all-gather run %d rank %d" % (it, r))
            assert dev["out"][r].guards_intact()
    g.destroy()
