"""Pins the CPU checker's reduce-copy against the mathematics (no GPU needed).

The reference holds no arithmetic, tests or golden vectors for this path, so the checker is
pinned by: exact-rational brute force with one rounding per fold step, cases whose answer
depends on the fold order, closed forms for int32 wraparound, and numpy's IEEE binary32 ops
as an independent implementation of each single step."""
import itertools
from fractions import Fraction

import numpy as np
import pytest

import helpers as H
import schedules as S


def _round_f32(q):
    """Exact rational -> nearest binary32 (ties to even), via Python's correctly rounded
    Fraction -> float (binary64) only when that is exact enough; done manually instead."""
    if q == 0:
        return np.float32(0.0)
    sign = -1 if q < 0 else 1
    a = abs(q)
    # find e with 2^e <= a < 2^(e+1)
    e = a.numerator.bit_length() - a.denominator.bit_length()
    if Fraction(2) ** e > a:
        e -= 1
    if Fraction(2) ** (e + 1) <= a:
        e += 1
    e = max(e, -126)  # subnormal spacing below 2^-126
    ulp = Fraction(2) ** (e - 23)
    n = a / ulp
    lo = n.numerator // n.denominator
    rem = n - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and lo % 2 == 1):
        lo += 1
    v = lo * ulp
    if v >= Fraction(2) ** 128:
        return np.float32(sign * np.inf)
    return np.float32(sign * float(v))  # v has <= 24 significant bits: exact in binary64


def _fold_exact(vals, compute):
    acc = Fraction(float(vals[0]))
    for x in vals[1:]:
        x = Fraction(float(x))
        if compute == "sum":
            acc = Fraction(float(_round_f32(acc + x)))
        elif compute == "prod":
            acc = Fraction(float(_round_f32(acc * x)))
        elif compute == "min":
            acc = x if x < acc else acc
        else:
            acc = x if acc < x else acc
    return np.float32(float(acc))


@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
@pytest.mark.parametrize("n_in", [2, 3, 8])
def test_f32_fold_matches_exact_rational(oracle, compute, n_in):
    count = 64
    lo, hi = (0.5, 2.0) if compute == "prod" else (-1.0, 1.0)
    ins = [oracle.fill_uniform_f32(count, 900 + n_in, k, lo, hi) for k in range(n_in)]
    # widen the dynamic range so that rounding actually happens in sums
    if compute == "sum":
        ins = [a * np.float32(10.0 ** (k % 4)) for k, a in enumerate(ins)]
    got = oracle.reduce("f32", compute, ins)
    want = np.array([_fold_exact([a[i] for a in ins], compute) for i in range(count)], dtype=np.float32)
    H.assert_bits_equal(got, want, "f32 %s n_in=%d" % (compute, n_in))


def test_fold_order_is_left_to_right(oracle):
    """(1e8 + 1) - 1e8 = 0 in binary32 when folded from the left; a tree or a right fold gives
    other answers for the permutations below."""
    big, one = np.float32(1e8), np.float32(1.0)
    cases = [
        ([big, one, -big], np.float32(0.0)),         # (1e8+1) rounds to 1e8
        ([big, -big, one], np.float32(1.0)),
        ([one, big, -big], np.float32(0.0)),
        ([np.float32(16777216.0), one, one], np.float32(16777216.0)),  # 2^24+1 ties to even, twice
        ([one, one, np.float32(16777216.0)], np.float32(16777218.0)),
    ]
    for vals, want in cases:
        ins = [np.full(3, v, dtype=np.float32) for v in vals]
        got = oracle.reduce("f32", "sum", ins)
        H.assert_bits_equal(got, np.full(3, want, dtype=np.float32), "order case %s" % (vals,))


def test_no_fused_multiply_add(oracle):
    """prod then sum must round in between: a*b+c with FMA would differ for these values.
    (Checked through two separate ops, as a collective step would issue them.)"""
    a = np.full(4, np.float32(1.0 + 2.0 ** -12), dtype=np.float32)
    p = oracle.reduce("f32", "prod", [a, a])                       # rounds 1 + 2^-11 + 2^-24
    H.assert_bits_equal(p, a * a, "product rounding")
    s = oracle.reduce("f32", "sum", [p, np.full(4, np.float32(-1.0), dtype=np.float32)])
    H.assert_bits_equal(s, np.full(4, np.float32(2.0 ** -11), dtype=np.float32), "sum after rounded product")


def test_i32_wraparound_closed_form(oracle):
    n_in, count = 5, 4096
    rng = np.random.default_rng(12)
    ins = [rng.integers(-2 ** 31, 2 ** 31, size=count, dtype=np.int64).astype(np.int32) for _ in range(n_in)]
    wide = [a.astype(object) for a in ins]
    want_sum = np.array([((sum(int(w[i]) for w in wide) + 2 ** 31) % 2 ** 32) - 2 ** 31 for i in range(count)], dtype=np.int64)
    H.assert_bits_equal(oracle.reduce("i32", "sum", ins), want_sum.astype(np.int32), "i32 sum mod 2^32")
    prod = [1] * count
    for w in wide:
        prod = [p * int(x) for p, x in zip(prod, w)]
    want_prod = np.array([((p + 2 ** 31) % 2 ** 32) - 2 ** 31 for p in prod], dtype=np.int64).astype(np.int32)
    H.assert_bits_equal(oracle.reduce("i32", "prod", ins), want_prod, "i32 prod mod 2^32")
    H.assert_bits_equal(oracle.reduce("i32", "max", ins), np.maximum.reduce(ins), "i32 max")
    H.assert_bits_equal(oracle.reduce("i32", "min", ins), np.minimum.reduce(ins), "i32 min")


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_half_types_accumulate_in_f32_round_once(oracle, dtype, compute):
    """Independent restatement with numpy: widen, fold step by step in binary32, narrow once.
    Differs from folding in the narrow type (checked to be a different answer somewhere)."""
    count, n_in = 20000, 8
    lo, hi = (0.5, 2.0) if compute == "prod" else (-4.0, 4.0)
    ins = [oracle.narrow(dtype, oracle.fill_uniform_f32(count, 77, k, lo, hi)) for k in range(n_in)]
    wide = [oracle.widen(dtype, a) for a in ins]
    acc = wide[0].copy()
    narrow_acc = wide[0].copy()
    for w in wide[1:]:
        if compute == "sum":
            acc = acc + w
            narrow_acc = oracle.widen(dtype, oracle.narrow(dtype, narrow_acc + w))
        elif compute == "prod":
            acc = acc * w
            narrow_acc = oracle.widen(dtype, oracle.narrow(dtype, narrow_acc * w))
        elif compute == "min":
            acc = np.where(w < acc, w, acc)
        else:
            acc = np.where(acc < w, w, acc)
    want = oracle.narrow(dtype, acc)
    got = oracle.reduce(dtype, compute, ins)
    H.assert_bits_equal(got, want, "%s %s" % (dtype, compute))
    if compute in ("sum", "prod"):
        assert not np.array_equal(got, oracle.narrow(dtype, narrow_acc)), \
            "rounding after every step would be indistinguishable on this input: weak test"


def test_copy_moves_bytes_unchanged(oracle):
    # signalling NaN patterns and every other 16-bit pattern survive a COPY
    allbits = np.arange(65536, dtype=np.uint16)
    H.assert_bits_equal(oracle.reduce("bf16", "sum", [allbits]), allbits, "bf16 copy")
    H.assert_bits_equal(oracle.reduce("f16", "max", [allbits]), allbits, "f16 copy")
    snan = np.array([0x7f800001, 0xff800001, 0x7fc00000], dtype=np.uint32).view(np.float32)
    H.assert_bits_equal(oracle.reduce("f32", "sum", [snan]), snan, "f32 copy keeps sNaN")


def test_multi_output_and_in_place(oracle):
    a = oracle.fill_uniform_f32(1000, 1, 0, -1, 1)
    b = oracle.fill_uniform_f32(1000, 1, 1, -1, 1)
    o1, o2 = np.empty_like(a), np.empty_like(a)
    oracle.reduce_copy("f32", "sum", [a, b], [o1, o2])
    H.assert_bits_equal(o1, a + b, "out 0")
    H.assert_bits_equal(o2, a + b, "out 1")
    b2 = b.copy()
    oracle.reduce_copy("f32", "sum", [a, b2], [b2])  # in place on input 1
    H.assert_bits_equal(b2, a + b, "in place")


def test_threaded_form_matches_scalar_form(oracle):
    for dtype in ("f32", "bf16", "i32"):
        ins = [H.gen(dtype, 300001, 5, k) for k in range(4)]
        want = oracle.reduce(dtype, "sum", ins)
        out = np.empty_like(ins[0])
        oracle.reduce_copy(dtype, "sum", ins, [out], nthreads=5)
        H.assert_bits_equal(out, want, "mt %s" % dtype)


def test_argument_checks(oracle):
    a = np.zeros(4, dtype=np.float32)
    with pytest.raises(ValueError):
        oracle.reduce_copy(99, "sum", [a], [a])
    with pytest.raises(ValueError):
        oracle.reduce_copy("f32", "sum", [a] * 9, [a])
    with pytest.raises(ValueError):
        oracle.reduce_copy("f32", "sum", [a], [])


# ---- DAG order (reference pccl/lang/utils/graph.py:94-112) ---------------------------------

def test_topo_sort_hand_worked(oracle):
    # diamond: dfs(0) -> 1 -> 3 (post: 3,1), then 2 (post: 2), then 0; reversed: 0,2,1,3
    assert oracle.topo_sort(4, [(0, 1), (0, 2), (1, 3), (2, 3)]) == [0, 2, 1, 3]
    # two roots; nodes visited in id order: dfs(0): 2 -> post 2,0 ; dfs(1): post 1 ; reversed 1,0,2
    assert oracle.topo_sort(3, [(0, 2), (1, 2)]) == [1, 0, 2]
    # chain given backwards by id: dfs(0) post 0; dfs(1): ->0 visited, post 1; dfs(2): post 2 => 2,1,0
    assert oracle.topo_sort(3, [(2, 1), (1, 0)]) == [2, 1, 0]
    # successor order is edge insertion order: 0->2 was added before 0->1
    assert oracle.topo_sort(3, [(0, 2), (0, 1)]) == [0, 1, 2]
    # isolated nodes: each is its own root, later roots come first after the reversal
    assert oracle.topo_sort(3, []) == [2, 1, 0]
    assert oracle.topo_sort(0, []) == []


def test_topo_sort_rejects_cycles_and_bad_ids(oracle):
    assert oracle.topo_sort(2, [(0, 1), (1, 0)]) is None   # graph.py:95-96 ValueError
    assert oracle.topo_sort(3, [(0, 1), (1, 2), (2, 1)]) is None
    assert oracle.topo_sort(1, [(0, 0)]) is None
    assert oracle.topo_sort(2, [(0, 2)]) is None           # graph.py:30-31 invalid node id


def test_topo_sort_respects_every_dependency(oracle):
    ops, _ = S.ring_allreduce_ops(8, [16, 32, 48])
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    pos = {op: i for i, op in enumerate(order)}
    assert sorted(order) == list(range(len(ops)))
    for i, o in enumerate(ops):
        for d in o["deps"]:
            assert pos[d] < pos[i]


# ---- ring all-reduce replay: invariants of the schedule itself -------------------------------

@pytest.mark.parametrize("world", [2, 3, 8])
def test_ring_schedule_is_an_allreduce(oracle, world):
    """All ranks end with identical bytes, and chunk c equals the left fold that starts at rank
    c and walks the ring, rounding to bf16 after every step (not one 8-way fp32 sum)."""
    sizes = [129, 1000]
    ops, per_rank = S.ring_allreduce_ops(world, sizes, dtype="bf16")
    assert len(ops) == 2 * world * (2 * world - 2)
    host_in = [H.gen("bf16", per_rank, 8, r) for r in range(world)]
    host_out = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    bufs = {"in": host_in, "out": host_out}
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs[b][r][e:e + n]), order)
    for r in range(1, world):
        H.assert_bits_equal(host_out[r], host_out[0], "rank %d vs 0" % r)
    off = 0
    for size in sizes:
        for c in range(world):
            sl = slice(off + c * size, off + (c + 1) * size)
            acc = host_in[c][sl]
            for step in range(1, world):
                acc = oracle.reduce("bf16", "sum", [acc, host_in[(c + step) % world][sl]])
            H.assert_bits_equal(host_out[0][sl], acc, "chunk %d" % c)
        off += world * size
    # a different but valid topological order gives the same bytes
    rev_out = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    bufs2 = {"in": host_in, "out": rev_out}
    memo = {}
    levels = sorted(range(len(ops)), key=lambda i: (len(_ancestors(ops, i, memo)), -i))
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs2[b][r][e:e + n]), levels)
    for r in range(world):
        H.assert_bits_equal(rev_out[r], host_out[r], "alternative order rank %d" % r)


def _ancestors(ops, i, memo):
    if i not in memo:
        s = set()
        for d in ops[i]["deps"]:
            s.add(d)
            s |= _ancestors(ops, d, memo)
        memo[i] = s
    return memo[i]


def test_u32_closed_form(oracle):
    """u32: arithmetic mod 2^32 in Python integers; min / max compare unsigned (the same bits as
    i32 give other answers as soon as a value exceeds 2^31)."""
    n_in, count = 5, 4096
    rng = np.random.default_rng(13)
    ins = [rng.integers(0, 2 ** 32, size=count, dtype=np.uint64).astype(np.uint32) for _ in range(n_in)]
    want_sum = np.array([sum(int(a[i]) for a in ins) % 2 ** 32 for i in range(count)], dtype=np.uint64).astype(np.uint32)
    H.assert_bits_equal(oracle.reduce("u32", "sum", ins), want_sum, "u32 sum mod 2^32")
    prod = [1] * count
    for a in ins:
        prod = [p * int(x) for p, x in zip(prod, a)]
    H.assert_bits_equal(oracle.reduce("u32", "prod", ins), np.array([p % 2 ** 32 for p in prod], dtype=np.uint64).astype(np.uint32),
                        "u32 prod mod 2^32")
    H.assert_bits_equal(oracle.reduce("u32", "max", ins), np.maximum.reduce(ins), "u32 max")
    H.assert_bits_equal(oracle.reduce("u32", "min", ins), np.minimum.reduce(ins), "u32 min")
    as_i32 = [a.view(np.int32) for a in ins]
    assert not np.array_equal(oracle.reduce("i32", "max", as_i32).view(np.uint32), oracle.reduce("u32", "max", ins))


def _round_f64(q):
    """Exact rational -> nearest binary64, ties to even: Python's Fraction -> float conversion
    is correctly rounded (it is integer division with round-half-even)."""
    return np.float64(float(q))


@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_f64_fold_matches_exact_rational(oracle, compute):
    count, n_in = 64, 5
    lo, hi = (0.5, 2.0) if compute == "prod" else (-1.0, 1.0)
    ins = [H.gen("f64", count, 910, k, kind="uniform", lo=lo, hi=hi) for k in range(n_in)]
    if compute == "sum":
        ins = [a * 10.0 ** (3 * (k % 4)) for k, a in enumerate(ins)]
    want = np.empty(count, dtype=np.float64)
    for i in range(count):
        acc = ins[0][i]
        for a in ins[1:]:
            x, y = Fraction(float(acc)), Fraction(float(a[i]))
            if compute == "sum":
                acc = _round_f64(x + y)
            elif compute == "prod":
                acc = _round_f64(x * y)
            elif compute == "min":
                acc = a[i] if a[i] < acc else acc
            else:
                acc = a[i] if acc < a[i] else acc
        want[i] = acc
    H.assert_bits_equal(oracle.reduce("f64", compute, ins), want, "f64 %s" % compute)


def test_f64_fold_order_and_width(oracle):
    """Answers that need a binary64 accumulator and a left fold: 2^53 + 1 + 1 stays 2^53 from
    the left (each +1 ties to even) and is 2^53 + 2 from the right; 1e8 + 1 - 1e8 is exactly 1
    in binary64 where binary32 loses it."""
    two53 = np.float64(2.0 ** 53)
    one = np.float64(1.0)
    for vals, want in (([two53, one, one], two53), ([one, one, two53], two53 + 2.0),
                       ([np.float64(1e8), one, np.float64(-1e8)], one)):
        ins = [np.full(3, v, dtype=np.float64) for v in vals]
        H.assert_bits_equal(oracle.reduce("f64", "sum", ins), np.full(3, want, dtype=np.float64), "f64 %s" % (vals,))


def test_normal_generator_threaded_form_and_shape(oracle):
    """fill_normal over several threads gives the bytes of the scalar loop (the generator is counter-based), and
    what it gives is a normal sample: mean, standard deviation, and tails at the rate the distribution has
    (a bounded stand-in such as a scaled uniform has none beyond 1.74 sigma)."""
    n = 1 << 20
    for dtype, sigma in (("f32", 1.0), ("bf16", 1e-2), ("f16", 1.0)):
        one = oracle.fill_normal(dtype, n, 9, 4, 0.0, sigma)
        many = oracle.fill_normal(dtype, n, 9, 4, 0.0, sigma, nthreads=5)
        assert np.array_equal(one, many)
        z = (oracle.widen(dtype, one) if dtype != "f32" else one).astype(np.float64) / sigma
        assert abs(z.mean()) < 5e-3 and abs(z.std() - 1.0) < 5e-3
        for k, rate in ((2.0, 4.55e-2), (3.0, 2.70e-3), (4.0, 6.33e-5)):
            seen = float((np.abs(z) > k).mean())
            assert 0.7 * rate < seen < 1.3 * rate, "%s: P(|z| > %g) = %g, a normal has %g" % (dtype, k, seen, rate)
    # another stream, another seed: other values
    assert not np.array_equal(oracle.fill_normal("f32", 64, 9, 4), oracle.fill_normal("f32", 64, 9, 5))
    assert not np.array_equal(oracle.fill_normal("f32", 64, 9, 4), oracle.fill_normal("f32", 64, 10, 4))
