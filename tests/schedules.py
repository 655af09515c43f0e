"""Test-side builders of op DAGs (ring all-reduce over virtual ranks resident on one GPU).

An op is a dict: dtype, compute, ins, outs, count, deps.  Operands are named symbolically as
(buffer, rank, element_offset); `materialise` turns them into addresses (device) or numpy views
(CPU checker).  The ring follows the textbook schedule: at reduce-scatter step s rank r folds
the partial sum of chunk (r - s) mod W coming from rank r-1 with its own copy of that chunk; at
all-gather step s it copies chunk (r - s + 1) mod W from rank r-1.  An op of (rank r, step l)
depends on the op of (rank r-1, step l-1), which also covers every write-after-read hazard
because going back W-1 steps along that rule reaches the reader of the overwritten chunk.
"""
import math


def ring_allreduce_ops(world, slice_sizes, dtype="bf16", compute="sum", base_elem=0):
    """slice_sizes[k] = elements per chunk of independent all-reduce k.
    Returns (ops, elems_per_rank).  Buffers: "in" (per-rank input), "out" (per-rank output)."""
    ops = []
    off = base_elem
    for size in slice_sizes:
        prev = {}
        for step in range(1, world):  # reduce-scatter
            cur = {}
            for r in range(world):
                c = (r - step) % world
                src_rank = (r - 1) % world
                incoming = ("in" if step == 1 else "out", src_rank, off + c * size)
                local = ("in", r, off + c * size)
                deps = [prev[src_rank]] if step > 1 else []
                ops.append(dict(dtype=dtype, compute=compute, ins=[incoming, local],
                                outs=[("out", r, off + c * size)], count=size, deps=deps))
                cur[r] = len(ops) - 1
            prev = cur
        for step in range(1, world):  # all-gather
            cur = {}
            for r in range(world):
                c = (r - step + 1) % world
                src_rank = (r - 1) % world
                ops.append(dict(dtype=dtype, compute=compute, ins=[("out", src_rank, off + c * size)],
                                outs=[("out", r, off + c * size)], count=size, deps=[prev[src_rank]]))
                cur[r] = len(ops) - 1
            prev = cur
        off += world * size
    return ops, off


def log_uniform_sizes(orc, n, seed, stream, lo_bytes, hi_bytes, elem_bytes):
    """n sizes in elements, log-uniform in [lo_bytes, hi_bytes], rounded down to whole elements."""
    out = []
    for i in range(n):
        u = (orc.rng_u64(seed, stream, i) >> 11) / float(1 << 53)
        b = lo_bytes * math.exp(u * math.log(hi_bytes / lo_bytes))
        out.append(max(1, int(b) // elem_bytes))
    return out


def materialise(ops, resolve):
    """resolve(buffer, rank, elem_offset, count) -> address or numpy view."""
    done = []
    for o in ops:
        d = dict(o)
        d["ins"] = [resolve(b, r, e, o["count"]) for (b, r, e) in o["ins"]]
        d["outs"] = [resolve(b, r, e, o["count"]) for (b, r, e) in o["outs"]]
        done.append(d)
    return done


def edges_of(ops):
    """(src, dst) pairs in the order CollectiveIR.create_operation adds them
    (reference pccl/lang/chunk.py:104-106: for each op, one edge per dependency)."""
    return [(d, i) for i, o in enumerate(ops) for d in o["deps"]]


def parse_schedule_text(text):
    """Test-side reader of the engine's schedule file (independent of the product parser).
    Returns (header dict, ops) with ops in the symbolic form used by `materialise`."""
    toks = []
    for line in text.splitlines():
        line = line.strip()
        if line and not line.startswith("#"):
            toks += line.split()
    it = iter(toks)

    def nxt():
        return next(it)

    assert nxt() == "pccl-schedule"
    version = int(nxt())
    assert version in (1, 2)
    hdr = {"version": version}
    for key in ("name", "dtype", "compute", "devices", "elems_per_device", "ops"):
        assert nxt() == key
        hdr[key] = nxt()
    for key in ("devices", "elems_per_device", "ops"):
        hdr[key] = int(hdr[key])
    ops = []
    for i in range(hdr["ops"]):
        assert nxt() == "op" and int(nxt()) == i
        kind, count = nxt(), int(nxt())
        assert nxt() == "deps"
        deps = [int(nxt()) for _ in range(int(nxt()))]
        if kind in ("NOTIFY", "GET_NOTIFIED"):
            assert nxt() == "slot"
            slot, parts = int(nxt()), 1
            if version >= 2:   # (version 2: the slots the signal takes, one per part of the data)
                assert nxt() == "parts"
                parts = int(nxt())
            ops.append(dict(signal=kind, slot=slot, parts=parts, value=count, ins=[], outs=[], count=0, deps=deps))
            continue
        sides = []
        for key in ("src", "dst"):
            assert nxt() == key
            sides.append([(nxt(), int(nxt()), int(nxt())) for _ in range(int(nxt()))])
        assert kind in ("COPY", "REDUCE")
        ops.append(dict(dtype=hdr["dtype"], compute=hdr["compute"], ins=sides[0], outs=sides[1], count=count, deps=deps))
    return hdr, ops


def replay_with_signals(oracle, ops, order, resolve):
    """CPU replay of a schedule that may hold signal ops: data ops go to the checker, NOTIFY
    records its value, GET_NOTIFIED asserts that the value it waits for has been published."""
    slots = {}
    for i in order:
        o = ops[i]
        if o.get("signal") == "NOTIFY":
            for w in range(o.get("parts", 1)):
                assert slots.get(o["slot"] + w, -1) < o["value"], "slot %d must rise" % (o["slot"] + w)
                slots[o["slot"] + w] = o["value"]
        elif o.get("signal") == "GET_NOTIFIED":
            for w in range(o.get("parts", 1)):
                assert slots.get(o["slot"] + w, -1) >= o["value"], "op %d waits for a value nobody published before it" % i
        else:
            oracle.reduce_copy(o["dtype"], o["compute"], [resolve(*x, o["count"]) for x in o["ins"]],
                               [resolve(*x, o["count"]) for x in o["outs"]])
    return slots


def random_pool_program(rng, pool_elems, n_ops):
    """Ops in program order over regions of one f32 pool.  Regions of equal length start at
    multiples of that length, sometimes pushed on by a few hundred elements, so that later ops
    meet earlier results at the same address, at a shifted address, or not at all.  Inside an
    op an output may be one of the inputs exactly; otherwise its operands are disjoint.
    Dependencies: every earlier op with a conflicting operand (RAW, WAW, WAR), transitively
    reduced, so that the program means what running the ops one after the other means and
    leans on whole-op dependencies being transitive."""
    lengths = [40_000, 40_000, 65_536, 100_000]
    ops = []
    for i in range(n_ops):
        n = lengths[rng.integers(len(lengths))]
        def region():
            base = int(rng.integers(0, (pool_elems - n - 1024) // n)) * n
            if rng.random() < 0.25:
                base += int(rng.integers(1, 8)) * 64
            return base
        def disjoint(a, b):
            return a + n <= b or b + n <= a
        n_in, n_out = int(rng.integers(1, 4)), int(rng.integers(1, 3))
        ins, outs = [], []
        while len(ins) < n_in:
            r = region()
            if all(disjoint(r, x) for x in ins):
                ins.append(r)
        while len(outs) < n_out:
            r = ins[0] if (not outs and rng.random() < 0.3) else region()
            if all(disjoint(r, x) for x in outs) and all(disjoint(r, x) or r == x for x in ins):
                outs.append(r)
        ops.append(dict(count=n, ins=ins, outs=outs, compute=["sum", "max", "min"][rng.integers(3)] if n_in > 1 else "sum"))
    def overlap(a, na, b, nb):
        return a < b + nb and b < a + na
    reach = []  # reach[i]: ops that op i transitively depends on
    for i, o in enumerate(ops):
        direct = []
        for j in range(i):
            p = ops[j]
            conflict = any(overlap(x, p["count"], y, o["count"]) for x in p["outs"] for y in o["ins"] + o["outs"]) or \
                any(overlap(x, p["count"], y, o["count"]) for x in p["ins"] for y in o["outs"])
            if conflict:
                direct.append(j)
        kept = [j for j in direct if not any(j in reach[k] for k in direct if k != j)]
        o["deps"] = kept
        reach.append(set(direct).union(*[reach[j] for j in direct]) if direct else set())
    return ops
