"""Seeded random sweep over everything a caller can vary at once: dtype, compute op, number of
inputs and outputs, element count (log-uniform, so the small counts around pack and workgroup
boundaries are as frequent as large ones), byte offsets of every buffer, an output aliasing an
input, and the three entry points (direct launch, queue executor, accumulate).  Every case is
compared bit for bit with the CPU checker, and the guard bands around every output are checked."""
import os

import numpy as np
import pytest

import helpers as H
import schedules as S

pytestmark = pytest.mark.gpu

# PCCL_TEST_SWEEP_SCALE=10 runs ten times as many cases from other seeds (a soak, not the default)
SCALE = max(1, int(os.environ.get("PCCL_TEST_SWEEP_SCALE", "1")))
SEED_SHIFT = 0 if SCALE == 1 else 7919

DTYPES = ["f32", "i32", "bf16", "f16", "f8e4m3", "f8e5m2", "f64", "u32"]
COMPUTES = ["sum", "prod", "min", "max"]


def _gen(dtype, compute, count, seed, k):
    if compute == "prod":
        if dtype == "i32":
            return H.gen(dtype, count, seed, k, lo=-7, hi=7)
        if dtype == "u32":
            return H.gen(dtype, count, seed, k, lo=0, hi=13)
        return H.gen(dtype, count, seed, k, kind="uniform", lo=0.5, hi=2.0)
    return H.gen(dtype, count, seed, k)


def _equal(oracle, dtype, got, want, what):
    if dtype in ("f8e4m3", "f8e5m2"):  # any NaN encoding of the format counts as NaN
        wn, gn = np.isnan(oracle.widen(dtype, want)), np.isnan(oracle.widen(dtype, got))
        assert np.array_equal(wn, gn), what + ": NaN positions"
        got, want = np.where(wn, 0, got), np.where(wn, 0, want)
    H.assert_bits_equal(got, want, what)


def _cases(seed, n):
    rng = np.random.default_rng(seed)
    for i in range(n):
        dtype = DTYPES[rng.integers(len(DTYPES))]
        compute = COMPUTES[rng.integers(len(COMPUTES))]
        es = H.ELEM_BYTES[dtype]
        count = int(np.exp(rng.uniform(0, np.log(300_000))))
        n_in, n_out = int(rng.integers(1, 9)), int(rng.integers(1, 9))
        aligned = rng.random() < 0.3
        offs = lambda m: [0 if aligned else int(rng.integers(0, 64 // es)) * es for _ in range(m)]
        yield i, dtype, compute, count, n_in, n_out, offs(n_in), offs(n_out), rng


@pytest.fixture
def restore_knobs(hip):
    yield
    hip.set_tuning(0, -1)
    hip.set_unroll(-1)
    hip.set_occupancy_lds(-1)


def _random_knobs(hip, rng):
    """Every second case forces a kernel variant that the built-in policy would only pick for
    much larger operands: cache treatment, packs per lane / lean kernel, persistent grid, LDS cap."""
    if rng.random() < 0.5:
        hip.set_tuning(0, -1)
        hip.set_unroll(-1)
        hip.set_occupancy_lds(-1)
        return "policy"
    mem, unroll = int(rng.integers(0, 3)), [-1, 0, 1, 4][rng.integers(4)]
    wg, lds = [0, 0, 1, 3][rng.integers(4)], [-1, 0, 32512, 65536][rng.integers(4)]
    hip.set_tuning(wg, mem)
    hip.set_unroll(unroll)
    hip.set_occupancy_lds(lds)
    return "mem=%d unroll=%d wg=%d lds=%d" % (mem, unroll, wg, lds)


def test_direct_launch_random(hip, oracle, restore_knobs):
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    for i, dtype, compute, count, n_in, n_out, in_offs, out_offs, rng in _cases(2024 + SEED_SHIFT, 600 * SCALE):
        knobs = _random_knobs(hip, rng)
        ins = [_gen(dtype, compute, count, 700 + i, k) for k in range(n_in)]
        want = oracle.reduce(dtype, compute, ins)
        what = "case %d: %s %s %d->%d count=%d in_offs=%s out_offs=%s [%s]" % (i, dtype, compute, n_in, n_out, count, in_offs, out_offs, knobs)
        d_in = [H.DevBuf(torch, dtype, count, off, src=a) for a, off in zip(ins, in_offs)]
        d_out = [H.DevBuf(torch, dtype, count, off) for off in out_offs]
        alias = rng.random() < 0.25      # output 0 is input k itself (in place)
        out_ptrs = [b.ptr for b in d_out]
        if alias:
            k = int(rng.integers(n_in))
            out_ptrs[0] = d_in[k].ptr
        hip.reduce_copy(dtype, compute, [b.ptr for b in d_in], out_ptrs, count, stream)
        torch.cuda.synchronize()
        for j in range(n_out):
            got = d_in[k].download() if (alias and j == 0) else d_out[j].download()
            _equal(oracle, dtype, got, want, what + " out %d%s" % (j, " (in place)" if alias and j == 0 else ""))
        for b in d_out + d_in:
            assert b.guards_intact(), what + ": wrote outside a buffer"


def test_queue_random(hip, oracle):
    """Graphs of 1..12 independent random ops each (mixed dtypes), random part sizes."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    gen = _cases(2025 + SEED_SHIFT, 300 * SCALE)
    g_no = 0
    while True:
        batch = []
        try:
            for _ in range(1 + g_no % 12):
                batch.append(next(gen))
        except StopIteration:
            pass
        if not batch:
            break
        ops, checks = [], []
        for i, dtype, compute, count, n_in, n_out, in_offs, out_offs, rng in batch:
            n_out = min(n_out, 10 - n_in)  # a queue op names at most 10 operands (payload of at most 255 bytes)
            out_offs = out_offs[:n_out]
            ins = [_gen(dtype, compute, count, 900 + i, k) for k in range(n_in)]
            d_in = [H.DevBuf(torch, dtype, count, off, src=a) for a, off in zip(ins, in_offs)]
            d_out = [H.DevBuf(torch, dtype, count, off) for off in out_offs]
            ops.append(dict(dtype=dtype, compute=compute, ins=[b.ptr for b in d_in], outs=[b.ptr for b in d_out], count=count))
            checks.append((dtype, oracle.reduce(dtype, compute, ins), d_out, d_in,
                           "graph %d op %d: %s %s %d->%d count=%d" % (g_no, len(ops) - 1, dtype, compute, n_in, n_out, count)))
        tile = [0, 1024, 4096, 16384][g_no % 4]
        g = hip.Graph(ops, tile_bytes=tile)
        g.run(stream)
        assert g.status(stream) == (len(ops), len(ops))
        for dtype, want, d_out, d_in, what in checks:
            for j, b in enumerate(d_out):
                _equal(oracle, dtype, b.download(), want, what + " out %d" % j)
                assert b.guards_intact(), what
        g.destroy()
        g_no += 1


def test_accumulate_random(hip, oracle, restore_knobs):
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    for i, dtype, compute, count, _, n_out, in_offs, out_offs, rng in _cases(2026 + SEED_SHIFT, 300 * SCALE):
        knobs = _random_knobs(hip, rng)
        src = _gen(dtype, compute, count, 1100 + i, 0)
        dsts = [_gen(dtype, compute, count, 1100 + i, 1 + j) for j in range(n_out)]
        d_src = H.DevBuf(torch, dtype, count, in_offs[0], src=src)
        d_dst = [H.DevBuf(torch, dtype, count, off, src=a) for a, off in zip(dsts, out_offs)]
        hip.accumulate(dtype, compute, d_src.ptr, [b.ptr for b in d_dst], count, stream)
        torch.cuda.synchronize()
        for j, b in enumerate(d_dst):
            _equal(oracle, dtype, b.download(), oracle.reduce(dtype, compute, [dsts[j], src]),
                   "case %d: %s %s 1->%d count=%d dst %d [%s]" % (i, dtype, compute, n_out, count, j, knobs))
            assert b.guards_intact()


# ---- random programs over one pool of memory ------------------------------------------------

def _run_pool_programs(hip, oracle, seeds, tile_auto=False):
    """Bytes only: the pool after every run equals sequential execution on the CPU.  Returns how many
    dependencies of each kind (whole-op, part by part) the executor reported."""
    import torch
    pool_elems = 2_000_000
    stream = torch.cuda.current_stream().cuda_stream
    kinds_seen = [0, 0]
    for seed in seeds:
        rng = np.random.default_rng(5000 + seed + SEED_SHIFT)
        prog = S.random_pool_program(rng, pool_elems, int(rng.integers(8, 60)))
        host = H.gen("f32", pool_elems, 777 + seed, 0, kind="uniform", lo=-1.0, hi=1.0)
        dev = H.DevBuf(torch, "f32", pool_elems, 0, src=host)
        tile = hip.TILE_AUTO if tile_auto else [0, 0, 16384, 65536][seed % 4]
        g = hip.Graph([dict(dtype="f32", compute=o["compute"], count=o["count"], deps=o["deps"],
                            ins=[dev.ptr + 4 * r for r in o["ins"]], outs=[dev.ptr + 4 * r for r in o["outs"]])
                       for o in prog], tile_bytes=tile)
        kinds = g.dependency_kinds()
        assert len(kinds) == sum(len(o["deps"]) for o in prog)
        kinds_seen[0] += kinds.count(0)
        kinds_seen[1] += kinds.count(1)
        for run in range(2):
            for o in prog:
                n = o["count"]
                oracle.reduce_copy("f32", o["compute"], [host[r:r + n].copy() for r in o["ins"]], [host[r:r + n] for r in o["outs"]])
            g.run(stream)
            done, total = g.status(stream)
            assert done == total == len(prog)
            H.assert_bits_equal(dev.download(), host, "seed %d run %d (%d ops, tile %d)" % (seed, run, len(prog), tile))
        assert dev.guards_intact()
        g.destroy()
    return kinds_seen


def test_random_programs_over_one_pool_match_sequential_execution(hip, oracle):
    """Programs whose ops alias each other's operands in every way the dependency analysis of
    the queue executor distinguishes: the pool after the run must equal, bit for bit, the pool
    after running the ops one by one on the CPU.  Each program runs twice (the second run
    starts from the first one's results and re-uses the re-armed graph)."""
    kinds_seen = _run_pool_programs(hip, oracle, range(6 * SCALE))
    # (plan shape, built-in settings only) the sweep met both kinds of dependency often
    assert min(kinds_seen) >= 20, kinds_seen


def _run_signal_programs(hip, oracle, seeds):
    """Bytes only.  Returns (signal ops carried by data ops, signal ops with entries of their own)."""
    import torch
    pool_elems = 1_000_000
    stream = torch.cuda.current_stream().cuda_stream
    carried_seen, own_seen = 0, 0
    for seed in seeds:
        rng = np.random.default_rng(8000 + seed + SEED_SHIFT)
        prog = S.random_pool_program(rng, pool_elems, int(rng.integers(6, 40)))
        host = H.gen("f32", pool_elems, 977 + seed, 0, kind="uniform", lo=-1.0, hi=1.0)
        dev = H.DevBuf(torch, "f32", pool_elems, 0, src=host)
        words = torch.zeros(1024, dtype=torch.int32, device="cuda")
        ops, new_index, n_words = [], {}, 0
        for i, o in enumerate(prog):
            deps = []
            for u in o["deps"]:
                if rng.random() < 0.5 and n_words < 1000:
                    word = words.data_ptr() + 4 * n_words
                    n_words += 1
                    ops.append(dict(primitive=2, signal=word, value=1, deps=[new_index[u]]))
                    ops.append(dict(primitive=3, signal=word, value=1, deps=[]))
                    deps.append(len(ops) - 1)
                else:
                    deps.append(new_index[u])
            new_index[i] = len(ops)
            ops.append(dict(dtype="f32", compute=o["compute"], count=o["count"], deps=deps,
                            ins=[dev.ptr + 4 * r for r in o["ins"]], outs=[dev.ptr + 4 * r for r in o["outs"]]))
        carrier = hip.plan_signals(ops)
        carried_seen += sum(1 for c in carrier if c >= 0)
        own_seen += sum(1 for k, c in enumerate(carrier) if c < 0 and ops[k].get("primitive", 0) >= 2)
        g = hip.Graph(ops, tile_bytes=[0, 16384, 65536][seed % 3])
        for run in range(3):
            for o in prog:
                n = o["count"]
                oracle.reduce_copy("f32", o["compute"], [host[r:r + n].copy() for r in o["ins"]], [host[r:r + n] for r in o["outs"]])
            g.run(stream)
            done, total = g.status(stream)
            assert done == total == len(ops)
            H.assert_bits_equal(dev.download(), host, "seed %d run %d (%d ops, %d words)" % (seed, run, len(ops), n_words))
        assert dev.guards_intact()
        g.destroy()
    return carried_seen, own_seen


def test_random_programs_with_dependencies_replaced_by_signal_words(hip, oracle):
    """The same kind of program with about half of its dependency edges u -> v replaced by
    NOTIFY(behind u) -> signal word -> GET_NOTIFIED(in front of v), a word per replaced edge: some of
    those signal ops ride on their data op, some (a second NOTIFY behind the same op, a second wait in
    front of it) queue entries of their own.  The pool must equal sequential execution, run after run."""
    carried_seen, own_seen = _run_signal_programs(hip, oracle, range(8 * SCALE))
    assert carried_seen >= 20 and own_seen >= 5, (carried_seen, own_seen)   # (plan shape, built-in settings only)


def _run_extra_edge_programs(hip, oracle, seeds):
    """Bytes only.  Returns (extra dependencies added, dependencies the executor meets part by part)."""
    import torch
    pool_elems = 1_500_000
    stream = torch.cuda.current_stream().cuda_stream
    extra, part_wise = 0, 0
    for seed in seeds:
        rng = np.random.default_rng(6100 + seed + SEED_SHIFT)
        prog = S.random_pool_program(rng, pool_elems, int(rng.integers(8, 50)))
        for i, o in enumerate(prog):
            for _ in range(2):
                if i and rng.random() < 0.4:
                    j = int(rng.integers(0, i))
                    if j not in o["deps"]:
                        o["deps"].append(j)
                        extra += 1
        host = H.gen("f32", pool_elems, 877 + seed, 0, kind="uniform", lo=-1.0, hi=1.0)
        dev = H.DevBuf(torch, "f32", pool_elems, 0, src=host)
        g = hip.Graph([dict(dtype="f32", compute=o["compute"], count=o["count"], deps=o["deps"],
                            ins=[dev.ptr + 4 * r for r in o["ins"]], outs=[dev.ptr + 4 * r for r in o["outs"]])
                       for o in prog], tile_bytes=[0, 16384, 65536][seed % 3])
        part_wise += g.dependency_kinds().count(1)
        for run in range(2):
            for o in prog:
                n = o["count"]
                oracle.reduce_copy("f32", o["compute"], [host[r:r + n].copy() for r in o["ins"]], [host[r:r + n] for r in o["outs"]])
            g.run(stream)
            done, total = g.status(stream)
            assert done == total == len(prog)
            H.assert_bits_equal(dev.download(), host, "seed %d run %d (%d ops)" % (seed, run, len(prog)))
        assert dev.guards_intact()
        g.destroy()
    return extra, part_wise


def test_random_programs_with_dependencies_between_ops_that_share_no_bytes(hip, oracle):
    """The same kind of program with extra dependencies that it does not need (to any earlier op): those
    between ops cut alike are met part by part, and the ops reached through them must still be looked at
    when a later op touches their bytes at another address.  The pool must equal sequential execution."""
    extra, part_wise = _run_extra_edge_programs(hip, oracle, range(6 * SCALE))
    assert extra >= 50 and part_wise >= 20, (extra, part_wise)   # (plan shape, built-in settings only)


# ---- the same sweeps under every documented switch of the executor: bytes only ---------------------

def _ring_through_the_queue(hip, oracle, world, size, seed, tile_auto=False):
    """Ring all-reduce over resident ranks as one graph (its chunks run as chains where chains are on)."""
    import torch
    from pccl_amd import lang
    stream = torch.cuda.current_stream().cuda_stream
    ir, per_rank = lang.ring_allreduce(world, size, dtype="bf16")
    low = ir.lower()
    host_in = [H.gen("bf16", per_rank, seed, r) for r in range(world)]
    bufs = {"in": [H.DevBuf(torch, "bf16", per_rank, 0, src=a) for a in host_in],
            "out": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(world)]}
    outs = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    hb = {"in": host_in, "out": outs}
    for o in low:
        n = o["count"]
        oracle.reduce_copy("bf16", "sum", [hb[b][r][e:e + n] for (b, r, e) in o["ins"]], [hb[b][r][e:e + n] for (b, r, e) in o["outs"]])
    g = hip.Graph(lang.bind(low, lambda b, r, e: bufs[b][r].ptr + 2 * e), tile_bytes=hip.TILE_AUTO if tile_auto else 0)
    for run in range(2):
        for r in range(world):
            bufs["out"][r].view().fill_(0xFF)
        g.run(stream)
        assert g.status(stream) == (len(low), len(low))
        for r in range(world):
            H.assert_bits_equal(bufs["out"][r].download(), outs[r], "ring %d x %d, run %d, rank %d" % (world, size, run, r))
            assert bufs["out"][r].guards_intact()
    g.destroy()


KNOBS = [("PCCL_HIP_PLAN_LAUNCHES", "0"), ("PCCL_HIP_ORDER_EDGES", "0"), ("PCCL_HIP_CHAINS", "0"), ("PCCL_HIP_CHAINS", "1m"),
         ("PCCL_HIP_CHAIN_BALANCE", "0"), ("PCCL_HIP_PART_DEPS", "0"), ("PCCL_HIP_FUSE_SIGNALS", "0"),
         ("PCCL_HIP_OWN_ENTRIES", "0"), ("PCCL_HIP_OWN_ENTRIES", "16"), ("PCCL_HIP_ORDER_BLOCK", "0"), ("PCCL_HIP_ORDER_BLOCK", "1"), ("PCCL_HIP_FOLD_COPIES", "0"),
         ("PCCL_HIP_LAST_LEVEL", "0"), ("PCCL_HIP_COUNT_ALL", "1"),
         ("PCCL_HIP_WIDE", "0"), ("PCCL_HIP_CHAIN_LAUNCH", "0"), ("PCCL_HIP_CHAIN_LAUNCH", "2")]


@pytest.mark.parametrize("name,value", KNOBS, ids=["%s=%s" % kv for kv in KNOBS])
def test_random_programs_under_each_executor_switch(hip, oracle, monkeypatch, name, value):
    """Every documented switch of the queue executor changes HOW a graph runs, never what it leaves in
    memory: a short form of the three random-program sweeps, a ring all-reduce whose chunks chain, one of
    uneven chunks, and graphs handed over with PCCL_HIP_TILE_AUTO, under each switch.  Bytes only; what the
    plan looks like under a switch is nobody's business here."""
    monkeypatch.setenv(name, value)
    _run_pool_programs(hip, oracle, range(3))
    _run_pool_programs(hip, oracle, range(3, 5), tile_auto=True)
    _run_signal_programs(hip, oracle, range(3))
    _run_extra_edge_programs(hip, oracle, range(3))
    _ring_through_the_queue(hip, oracle, 8, 20_011, 3100)
    _ring_through_the_queue(hip, oracle, 4, 300_007, 3101)
    _ring_through_the_queue(hip, oracle, 4, 1_501, 3102, tile_auto=True)
