"""Schedule emitters: collectives written against :class:`CollectiveIR`.

The reference reserves ``pccl/lang/operator.py`` and ``example/collective/allreduce.py`` for
this and leaves both empty, so the schedules are this build's.
"""
import math

from .ir import Chunk, CollectiveIR, Device, DeviceType, Link, PrimitiveOpType


# element sizes of the dtype names the device plugin registers
ELEM_BYTES = {"f64": 8, "f32": 4, "i32": 4, "u32": 4, "bf16": 2, "f16": 2, "f8e4m3": 1, "f8e5m2": 1}


def _ring_ir(name, world, dtype, compute):
    ir = CollectiveIR(name, dtype=dtype, compute=compute)
    for r in range(world):
        ir.add_device(Device(r, DeviceType.ROCM, memory_bandwidth=8.0e12, compute_capability=9.5))
    for r in range(world):
        if world > 1 and (world > 2 or r == 0):
            ir.add_link(Link(r, (r + 1) % world, bandwidth=153.0e9, latency=1.0e-6))
    return ir


def ring_allreduce(world, chunk_elems, dtype="bf16", compute="sum", name="ring_allreduce", ir=None, base=0):
    """Out-of-place ring all-reduce of `world` chunks of `chunk_elems` elements per rank.

    Buffers: "in" (each rank's contribution) and "out" (each rank's result), chunk c of a rank
    at element offset base + c*chunk_elems.  Reduce-scatter step s (1..W-1): rank r folds the
    partial sum of chunk (r-s) mod W held by rank r-1 with its own contribution.  All-gather
    step s: rank r copies chunk (r-s+1) mod W from rank r-1.  The op of (rank r, level l)
    depends on the op of (rank r-1, level l-1); following that rule back W-1 levels reaches the
    last reader of every location an op overwrites, so no other edges are needed.
    Returns (ir, elements_per_rank_used)."""
    W = world
    ir = ir or _ring_ir(name, W, dtype, compute)
    prev = {}
    for step in range(1, W):
        cur = {}
        for r in range(W):
            c, p = (r - step) % W, (r - 1) % W
            off = base + c * chunk_elems
            incoming = ("in" if step == 1 else "out", p, off)
            ranks = {(c + i) % W for i in range(step + 1)}
            cur[r] = ir.create_operation(
                PrimitiveOpType.REDUCE,
                src_chunk=Chunk(ranks - {r}, p, chunk_elems, off), tgt_chunk=Chunk(ranks, r, chunk_elems, off),
                src_device=p, tgt_device=r, dependencies=[prev[p]] if step > 1 else [],
                metadata={"srcs": [incoming, ("in", r, off)], "tgt_buffer": "out", "level": step})
        prev = cur
    full = set(range(W))
    for step in range(1, W):
        cur = {}
        for r in range(W):
            c, p = (r - step + 1) % W, (r - 1) % W
            off = base + c * chunk_elems
            cur[r] = ir.create_operation(
                PrimitiveOpType.COPY,
                src_chunk=Chunk(full, p, chunk_elems, off), tgt_chunk=Chunk(full, r, chunk_elems, off),
                src_device=p, tgt_device=r, dependencies=[prev[p]],
                metadata={"src_buffer": "out", "tgt_buffer": "out", "level": W - 1 + step})
        prev = cur
    return ir, base + W * chunk_elems


def ring_reduce_scatter(world, chunk_elems, dtype="bf16", compute="sum", name="ring_reduce_scatter"):
    """The reduce-scatter half of the ring: after W-1 steps rank r holds, in "out" at chunk
    (r+1) mod W, the fold of that chunk over all ranks (in ring order starting at the chunk's
    own rank).  Other chunks of "out" are partial sums or untouched.  Returns (ir, elems)."""
    W = world
    ir = _ring_ir(name, W, dtype, compute)
    prev = {}
    for step in range(1, W):
        cur = {}
        for r in range(W):
            c, p = (r - step) % W, (r - 1) % W
            off = c * chunk_elems
            incoming = ("in" if step == 1 else "out", p, off)
            ranks = {(c + i) % W for i in range(step + 1)}
            cur[r] = ir.create_operation(
                PrimitiveOpType.REDUCE,
                src_chunk=Chunk(ranks - {r}, p, chunk_elems, off), tgt_chunk=Chunk(ranks, r, chunk_elems, off),
                src_device=p, tgt_device=r, dependencies=[prev[p]] if step > 1 else [],
                metadata={"srcs": [incoming, ("in", r, off)], "tgt_buffer": "out", "level": step})
        prev = cur
    return ir, W * chunk_elems


def ring_all_gather(world, chunk_elems, dtype="bf16", name="ring_all_gather"):
    """Rank r contributes chunk r of its "in"; afterwards every rank's "out" holds all W chunks.
    Level 1: every rank copies its own chunk in -> out; levels 2..W: rank r copies chunk
    (r-s+1) mod W from rank r-1's "out".  Returns (ir, elems)."""
    W = world
    ir = _ring_ir(name, W, dtype, "sum")
    prev = {}
    for r in range(W):
        off = r * chunk_elems
        prev[r] = ir.create_operation(
            PrimitiveOpType.COPY, src_chunk=Chunk({r}, r, chunk_elems, off), tgt_chunk=Chunk({r}, r, chunk_elems, off),
            src_device=r, tgt_device=r, dependencies=[], metadata={"src_buffer": "in", "tgt_buffer": "out", "level": 1})
    for step in range(1, W):
        cur = {}
        for r in range(W):
            c, p = (r - step) % W, (r - 1) % W
            off = c * chunk_elems
            cur[r] = ir.create_operation(
                PrimitiveOpType.COPY, src_chunk=Chunk({c}, p, chunk_elems, off), tgt_chunk=Chunk({c}, r, chunk_elems, off),
                src_device=p, tgt_device=r, dependencies=[prev[p]],
                metadata={"src_buffer": "out", "tgt_buffer": "out", "level": 1 + step})
        prev = cur
    return ir, W * chunk_elems


def direct_allreduce(world, slice_elems, dtype="bf16", compute="sum", name="direct_allreduce"):
    """The one-exchange all-reduce for a fully connected node: rank d folds slice d of all W
    "in" buffers in rank order (one W-input REDUCE, W <= 8), then one COPY stores the result
    into the other ranks' "out" (W-1 destinations).  Same ops as the native generator
    ``pccl_schedule_write_direct_allreduce``.  Returns (ir, elems)."""
    W = world
    if W > 8:
        raise ValueError("direct all-reduce folds one input per rank: at most 8 ranks")
    ir = _ring_ir(name, W, dtype, compute)
    full = set(range(W))
    for d in range(W):
        off = d * slice_elems
        red = ir.create_operation(
            PrimitiveOpType.REDUCE if W > 1 else PrimitiveOpType.COPY,
            src_chunk=Chunk(full, d, slice_elems, off), tgt_chunk=Chunk(full, d, slice_elems, off),
            src_device=d, tgt_device=d, dependencies=[],
            metadata={"srcs": [("in", r, off) for r in range(W)], "src_buffer": "in", "tgt_buffer": "out", "level": 1})
        if W > 1:
            others = [r for r in range(W) if r != d]
            ir.create_operation(
                PrimitiveOpType.COPY, src_chunk=Chunk(full, d, slice_elems, off), tgt_chunk=Chunk(full, others[0], slice_elems, off),
                src_device=d, tgt_device=others[0], dependencies=[red],
                metadata={"src_buffer": "out", "tgt_buffer": "out", "dsts": [("out", r, off) for r in others[1:]], "level": 2})
    return ir, W * slice_elems


def broadcast(world, elems, root=0, dtype="bf16", name="broadcast"):
    """Root's "in" to every rank's "out": one COPY with W destinations (W <= 8)."""
    W = world
    if W > 8:
        raise ValueError("one COPY names at most 8 destinations")
    ir = _ring_ir(name, W, dtype, "sum")
    full = {root}
    others = [r for r in range(W) if r != root]
    ir.create_operation(
        PrimitiveOpType.COPY, src_chunk=Chunk(full, root, elems, 0), tgt_chunk=Chunk(full, root, elems, 0),
        src_device=root, tgt_device=root, dependencies=[],
        metadata={"src_buffer": "in", "tgt_buffer": "out", "dsts": [("out", r, 0) for r in others], "level": 1})
    return ir, elems


def all_to_all(world, chunk_elems, dtype="bf16", name="all_to_all"):
    """Rank r's "in" chunk d goes to rank d's "out" chunk r: W*W independent COPY ops (the
    diagonal ones stay on their rank)."""
    W = world
    ir = _ring_ir(name, W, dtype, "sum")
    for r in range(W):
        for d in range(W):
            ir.create_operation(
                PrimitiveOpType.COPY, src_chunk=Chunk({r}, r, chunk_elems, d * chunk_elems),
                tgt_chunk=Chunk({r}, d, chunk_elems, r * chunk_elems), src_device=r, tgt_device=d, dependencies=[],
                metadata={"src_buffer": "in", "tgt_buffer": "out", "level": 1})
    return ir, W * chunk_elems


def ring_allreduce_signalled(world, chunk_elems, dtype="bf16", compute="sum", name="ring_allreduce_signalled",
                             first_slot=0, signal_parts=1):
    """The same ring all-reduce written the way ranks on different GPUs have to write it:
    dependency edges only between ops of one rank; the hand-over between neighbours goes
    NOTIFY (producer) -> signal slot -> GET_NOTIFIED (consumer).  Link (r-1) -> r uses slot
    first_slot + r, and the value is the step number, so every slot sees its values rise.
    signal_parts = K >= 2: every signal is K slots, one per part of the chunk it announces (link
    (r-1) -> r: slots first_slot + r * K ...), so that a rank starts on part p of a step as soon as its
    neighbour has finished part p of the step before (schedule format version 2).
    Returns (ir, elements_per_rank_used)."""
    W = world
    K = max(1, int(signal_parts))
    if first_slot + W * K > 256:
        raise ValueError("%d links of %d slots each do not fit the 256 signal slots" % (W, K))
    ir = _ring_ir(name, W, dtype, compute)
    last = {}  # rank -> its latest op
    for step in range(1, 2 * W - 1):
        reduce_phase = step < W
        for r in range(W):
            p = (r - 1) % W
            c = (r - step) % W if reduce_phase else (r - (step - (W - 1)) + 1) % W
            off = c * chunk_elems
            deps = [last[r]] if r in last else []
            if step > 1:
                whole = Chunk(set(), p, chunk_elems, off)
                deps = [ir.create_operation(PrimitiveOpType.GET_NOTIFIED, src_chunk=whole, tgt_chunk=whole, src_device=p,
                                            tgt_device=r, dependencies=deps,
                                            metadata={"slot": first_slot + r * K, "value": step - 1, "parts": K})]
            if reduce_phase:
                ranks = {(c + i) % W for i in range(step + 1)}
                op = ir.create_operation(
                    PrimitiveOpType.REDUCE, src_chunk=Chunk(ranks - {r}, p, chunk_elems, off),
                    tgt_chunk=Chunk(ranks, r, chunk_elems, off), src_device=p, tgt_device=r, dependencies=deps,
                    metadata={"srcs": [("in" if step == 1 else "out", p, off), ("in", r, off)], "tgt_buffer": "out"})
            else:
                full = set(range(W))
                op = ir.create_operation(
                    PrimitiveOpType.COPY, src_chunk=Chunk(full, p, chunk_elems, off), tgt_chunk=Chunk(full, r, chunk_elems, off),
                    src_device=p, tgt_device=r, dependencies=deps, metadata={"src_buffer": "out", "tgt_buffer": "out"})
            done = Chunk(set(), r, chunk_elems, off)
            last[r] = ir.create_operation(PrimitiveOpType.NOTIFY, src_chunk=done, tgt_chunk=done, src_device=r,
                                          tgt_device=(r + 1) % W, dependencies=[op],
                                          metadata={"slot": first_slot + ((r + 1) % W) * K, "value": step, "parts": K})
    return ir, W * chunk_elems


def ring_rank_share(world, chunk_elems, dtype="bf16", compute="sum", name="ring_rank_share", gather_buffers_of_their_own=False):
    """ONE rank's share of a ring all-reduce at world size `world`, its peers standing in as buffers: W - 1
    reduce-copy steps (incoming chunk + local chunk -> output chunk + send buffer) and W - 1 copy steps
    (incoming reduced chunk -> output chunk).  Step s of the first phase works on chunk (W - 1 - s) mod W, step s
    of the second on chunk (W - s) mod W.

    Regions ("devices" of the schedule file, each W * chunk_elems elements of the "in" and the "out" tensor):
    0 = the rank itself ("in": its gradient, W chunks; "out": the result), 1 = what arrives from the neighbour
    ("in": chunk s = the incoming buffer of step s; "out" chunk 0: the send buffer), and, with
    gather_buffers_of_their_own, 2 = a second set of incoming buffers that the copy steps read (otherwise copy step
    s reads the incoming buffer of reduce step s again).
    Dependencies are the hazards of the buffers: every reduce step writes the one send buffer (step s behind step
    s - 1), and copy step s overwrites the output chunk that reduce step s - 1 wrote.
    Returns (ir, elements_per_region)."""
    W, n = world, chunk_elems
    ir = CollectiveIR(name, dtype=dtype, compute=compute)
    for d in range(3 if gather_buffers_of_their_own else 2):
        ir.add_device(Device(d, DeviceType.ROCM, memory_bandwidth=8.0e12, compute_capability=9.5))
    reduce_ops = []
    for s in range(W - 1):
        c = (W - 1 - s) % W
        reduce_ops.append(ir.create_operation(
            PrimitiveOpType.REDUCE, src_chunk=Chunk({1}, 1, n, s * n), tgt_chunk=Chunk({0, 1}, 0, n, c * n), src_device=1, tgt_device=0,
            dependencies=[reduce_ops[-1]] if reduce_ops else [],
            metadata={"srcs": [("in", 1, s * n), ("in", 0, c * n)], "tgt_buffer": "out", "dsts": [("out", 1, 0)]}))
    src_region = 2 if gather_buffers_of_their_own else 1
    for s in range(W - 1):
        c = (W - s) % W
        ir.create_operation(
            PrimitiveOpType.COPY, src_chunk=Chunk({0, 1}, src_region, n, s * n), tgt_chunk=Chunk({0, 1}, 0, n, c * n),
            src_device=src_region, tgt_device=0, dependencies=[reduce_ops[s - 1]] if s else [],
            metadata={"src_buffer": "in", "tgt_buffer": "out"})
    return ir, W * n


def log_uniform_sizes(n, seed, lo_bytes, hi_bytes, elem_bytes):
    """n sizes in elements, log-uniform in [lo_bytes, hi_bytes] (splitmix64 stream of `seed`)."""
    def mix(z):
        z &= (1 << 64) - 1
        z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & ((1 << 64) - 1)
        z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & ((1 << 64) - 1)
        return z ^ (z >> 31)
    sizes = []
    for i in range(n):
        u = (mix(seed * 0x9e3779b97f4a7c15 + (i + 1) * 0x9e3779b97f4a7c15) >> 11) / float(1 << 53)
        sizes.append(max(1, int(lo_bytes * math.exp(u * math.log(hi_bytes / lo_bytes))) // elem_bytes))
    return sizes


def small_message_allreduce(world=8, n_slices=36, n_extra=64, seed=4, lo_bytes=8 << 10, hi_bytes=256 << 10,
                            dtype="bf16", compute="sum"):
    """The small-message program: `n_slices` independent ring all-reduces whose chunk sizes
    are log-uniform in [lo_bytes, hi_bytes] (one draw per slice: the 2*(W-1)*W ops of a slice
    share it), plus `n_extra` independent level-1 COPY ops in -> out with sizes drawn the same
    way.  world=8, 36 slices, 64 extras: 36*112 + 64 = 4096 ops, DAG depth 14.
    Returns (ir, elements_per_rank)."""
    es = ELEM_BYTES[dtype]
    sizes = log_uniform_sizes(n_slices + n_extra, seed, lo_bytes, hi_bytes, es)
    ir = _ring_ir("small_message_allreduce", world, dtype, compute)
    base = 0
    for k in range(n_slices):
        ir, base = ring_allreduce(world, sizes[k], dtype, compute, ir=ir, base=base)
    # extras: rank i % W copies a private region; regions of one round share an offset
    for i in range(n_extra):
        r, n = i % world, sizes[n_slices + i]
        full = {r}
        ir.create_operation(PrimitiveOpType.COPY, src_chunk=Chunk(full, r, n, base), tgt_chunk=Chunk(full, r, n, base),
                            src_device=r, tgt_device=r, dependencies=[],
                            metadata={"src_buffer": "in", "tgt_buffer": "out", "level": 1})
        if r == world - 1 or i == n_extra - 1:
            base += max(sizes[n_slices + i - r:n_slices + i + 1])
    return ir, base


def bind(lowered, resolve, signals=None):
    """Replaces symbolic operands: resolve(buffer, device, element_offset) -> address.
    Signal ops get "signal" = signals + 4 * slot (signals: address of the int slot array); "parts" stays."""
    out = []
    for o in lowered:
        d = dict(o)
        if o.get("primitive", 0) >= 2:
            if signals is None:
                raise ValueError("schedule has signal ops: pass the address of the signal slots")
            d["signal"] = int(signals) + 4 * o["slot"]
            out.append(d)
            continue
        d["ins"] = [resolve(*x) for x in o["ins"]]
        d["outs"] = [resolve(*x) for x in o["outs"]]
        out.append(d)
    return out
