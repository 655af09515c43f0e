"""The rule that lets a dependency be met part by part (pccl_hip_classify_dependencies, host
only) against every order of execution it allows: a CPU model of the queue executor runs the
parts of random programs in adversarial random orders, and the memory afterwards must equal
what running the ops one after the other leaves, bit for bit."""
import numpy as np
import pytest

import schedules as S
from pccl_amd import hip

BASE = 0x7f0000000000  # any address: the rule only compares operand addresses


def _ops_for_abi(prog):
    return [dict(dtype="f32", compute=o["compute"], count=o["count"], deps=o["deps"],
                 ins=[BASE + 4 * r for r in o["ins"]], outs=[BASE + 4 * r for r in o["outs"]]) for o in prog]


def _fold(compute, xs):
    acc = xs[0]
    for x in xs[1:]:
        acc = {"sum": np.add, "max": np.maximum, "min": np.minimum}[compute](acc, x)
    return acc


def _sequential(prog, pool):
    for o in prog:
        n = o["count"]
        r = _fold(o["compute"], [pool[x:x + n].copy() for x in o["ins"]])
        for y in o["outs"]:
            pool[y:y + n] = r
    return pool


def _executor_model(prog, parts, kinds, pool, rng, eager):
    """Runs every (op, part) once, in a random order among those the executor would allow:
    a part may run when every whole-op dependency of its op is complete and part p of every
    part-by-part dependency is done.  `eager`: probability of picking the runnable part of the
    LATEST op (drives successors as far ahead of their predecessors as the rule lets them)."""
    n_ops = len(prog)
    done_parts = [set() for _ in range(n_ops)]
    kind_of, at = [], 0
    for o in prog:
        kind_of.append(kinds[at:at + len(o["deps"])])
        at += len(o["deps"])
    pending = {(i, p) for i in range(n_ops) for p in range(parts[i])}
    def runnable(i, p):
        for d, k in zip(prog[i]["deps"], kind_of[i]):
            if k:
                if p not in done_parts[d]:
                    return False
            elif len(done_parts[d]) != parts[d]:
                return False
        return True
    while pending:
        ready = sorted(x for x in pending if runnable(*x))
        assert ready, "executor model is stuck"
        i, p = ready[-1] if rng.random() < eager else ready[rng.integers(len(ready))]
        o = prog[i]
        per = hip.part_elems(o["count"], parts[i])
        lo, hi = p * per, min((p + 1) * per, o["count"])
        if lo < hi:
            r = _fold(o["compute"], [pool[x + lo:x + hi].copy() for x in o["ins"]])
            for y in o["outs"]:
                pool[y + lo:y + hi] = r
        done_parts[i].add(p)
        pending.remove((i, p))
    return pool


def _naive_kinds(prog, parts):
    """What the rule must NOT be: part by part whenever two ops are merely cut alike."""
    return [1 if (prog[d]["count"] == o["count"] and parts[d] == parts[i] and parts[i] > 1) else 0
            for i, o in enumerate(prog) for d in o["deps"]]


def _program(seed):
    rng = np.random.default_rng(9000 + seed)
    pool_elems = 600_000
    prog = S.random_pool_program(rng, pool_elems, int(rng.integers(6, 28)))
    parts = [max(1, -(-o["count"] * 4 // 65536)) for o in prog]
    pool = rng.uniform(-1, 1, pool_elems).astype(np.float32)
    return rng, prog, parts, pool


def test_rule_is_sound_under_adversarial_orders():
    seen = [0, 0]
    for seed in range(100):
        rng, prog, parts, pool = _program(seed)
        kinds = hip.classify_dependencies(_ops_for_abi(prog), parts)
        assert len(kinds) == sum(len(o["deps"]) for o in prog)
        seen[0] += kinds.count(0)
        seen[1] += kinds.count(1)
        want = _sequential(prog, pool.copy())
        for eager in (1.0, 0.7, 0.0):
            got = _executor_model(prog, parts, kinds, pool.copy(), rng, eager)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "seed %d eager %.1f" % (seed, eager)
    assert min(seen) >= 100, seen  # both kinds of dependency were met often


def test_rule_is_sound_with_dependencies_between_ops_that_share_no_bytes():
    """Dependencies the program does not need (to any earlier op, conflict or not) are met part by part
    where the ops are cut alike; what matters is that ops reached only through such edges are still looked
    at when a later op touches their bytes at another address."""
    extra = 0
    for seed in range(200, 300):
        rng, prog, parts, pool = _program(seed)
        for i, o in enumerate(prog):
            if i and rng.random() < 0.5:
                j = int(rng.integers(0, i))
                if j not in o["deps"]:
                    o["deps"].append(j)
                    extra += 1
        kinds = hip.classify_dependencies(_ops_for_abi(prog), parts)
        want = _sequential(prog, pool.copy())
        for eager in (1.0, 0.7, 0.0):
            got = _executor_model(prog, parts, kinds, pool.copy(), rng, eager)
            assert np.array_equal(got.view(np.uint32), want.view(np.uint32)), "seed %d eager %.1f" % (seed, eager)
    assert extra >= 300, extra


def test_the_model_catches_an_unsound_rule():
    """Teeth: with 'cut alike' as the only condition some order gives different memory."""
    caught = 0
    for seed in range(100, 140):
        rng, prog, parts, pool = _program(seed)
        want = _sequential(prog, pool.copy())
        got = _executor_model(prog, parts, _naive_kinds(prog, parts), pool.copy(), rng, 1.0)
        caught += not np.array_equal(got.view(np.uint32), want.view(np.uint32))
    assert caught >= 5, caught


def test_rule_special_cases():
    n = 100_000
    def op(ins, outs, deps, count=n):
        return dict(dtype="f32", compute="sum", count=count, deps=deps, ins=[BASE + 4 * r for r in ins],
                    outs=[BASE + 4 * r for r in outs])
    A = op([0, n], [2 * n], [])
    # same address, cut alike: part by part; one part only: nothing to gain, whole-op
    assert hip.classify_dependencies([A, op([2 * n, n], [3 * n], [0])], [4, 4]) == [1]
    assert hip.classify_dependencies([A, op([2 * n, n], [3 * n], [0])], [1, 1]) == [0]
    # cut differently, or different lengths
    assert hip.classify_dependencies([A, op([2 * n, n], [3 * n], [0])], [4, 5]) == [0]
    assert hip.classify_dependencies([A, op([2 * n, n], [3 * n], [0], count=n - 64)], [4, 4]) == [0]
    # shifted overlap: whole-op; no overlap at all (the caller orders two ops that share no bytes): part by part
    assert hip.classify_dependencies([A, op([2 * n + 64, n], [4 * n], [0])], [4, 4]) == [0]
    assert hip.classify_dependencies([A, op([5 * n, n], [6 * n], [0])], [4, 4]) == [1]
    assert hip.classify_dependencies([A, op([5 * n, n], [6 * n], [0])], [4, 5]) == [0]
    # write-after-read and write-after-write at the same address
    assert hip.classify_dependencies([A, op([5 * n, 6 * n], [0], [0])], [4, 4]) == [1]
    assert hip.classify_dependencies([A, op([5 * n, 6 * n], [2 * n], [0])], [4, 4]) == [1]
    # an ancestor reached only through part-by-part edges is read at a shifted address
    X = op([0, n], [10 * n], [])
    mid = op([10 * n, n], [3 * n], [0])
    assert hip.classify_dependencies([X, mid, op([3 * n, 10 * n + 64], [7 * n], [1])], [4, 4, 4]) == [1, 0]
    # ... which does not matter when the edge in between is whole-op anyway
    mid_whole = op([10 * n + 64, n], [3 * n], [0])
    assert hip.classify_dependencies([X, mid_whole, op([3 * n, 10 * n + 64], [7 * n], [1])], [4, 4, 4]) == [0, 1]
    # errors: cycle, bad dependency
    with pytest.raises(hip.PcclError):
        hip.classify_dependencies([op([0, n], [2 * n], [1]), op([2 * n, n], [3 * n], [0])], [4, 4])
    with pytest.raises(hip.PcclError):
        hip.classify_dependencies([op([0, n], [2 * n], [3])], [4])
