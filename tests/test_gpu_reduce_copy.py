"""GPU parity: pccl_hip_reduce_copy (through the C ABI) against the CPU checker."""
import itertools

import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

COUNTS_SMALL = [1, 2, 3, 7, 8, 15, 16, 17, 63, 64, 65, 127, 255, 256, 257, 1023, 1024, 1025, 4099, 65537]


def _inputs(dtype, compute, n_in, count, seed):
    if compute == "prod":
        if dtype == "u32":
            return [H.gen(dtype, count, seed, k, lo=0, hi=13) for k in range(n_in)]
        return [H.gen(dtype, count, seed, k, kind="uniform", lo=0.5, hi=2.0) if dtype != "i32"
                else H.gen(dtype, count, seed, k, lo=-7, hi=7) for k in range(n_in)]
    if dtype in ("i32", "u32"):
        return [H.gen(dtype, count, seed, k) for k in range(n_in)]
    return [H.gen(dtype, count, seed, k, kind="normal") for k in range(n_in)]


def test_config1_f32_sum_2in(hip, oracle):
    """fp32 sum of 2 inputs, 1,048,576 elements, uniform[-1,1) seed 0, aligned; bit-exact."""
    import torch
    n = 1 << 20
    ins = [oracle.fill_uniform_f32(n, 0, k, -1.0, 1.0) for k in range(2)]
    want = oracle.reduce("f32", "sum", ins)
    (got,) = H.hip_reduce(torch, hip, "f32", "sum", ins)
    H.assert_bits_equal(got, want, "config 1")
    # and the checker itself agrees with numpy's IEEE add on this case
    H.assert_bits_equal(want, ins[0] + ins[1], "oracle vs numpy")


@pytest.mark.parametrize("dtype", ["f32", "i32", "bf16", "f16", "f64", "u32"])
@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_all_dtype_op_nin(hip, oracle, dtype, compute):
    """Every (dtype, compute, n_in) instantiation on ragged counts, aligned buffers."""
    import torch
    for n_in in range(1, 9):
        for count in (1, 5, 257, 4099, 70001):
            ins = _inputs(dtype, compute, n_in, count, seed=100 + n_in)
            want = oracle.reduce(dtype, compute, ins)
            (got,) = H.hip_reduce(torch, hip, dtype, compute, ins)
            H.assert_bits_equal(got, want, "%s %s n_in=%d count=%d" % (dtype, compute, n_in, count))


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f64"])
def test_small_counts_every_offset(hip, oracle, dtype):
    """Counts around pack / wavefront / workgroup boundaries at every element offset of output 0."""
    import torch
    es = H.ELEM_BYTES[dtype]
    for count in COUNTS_SMALL:
        ins = _inputs(dtype, "sum", 3, count, seed=7)
        want = oracle.reduce(dtype, "sum", ins)
        for off in range(0, 64, es):
            in_offs = [(off + 4 * k * es) % 64 for k in range(3)]
            (got,) = H.hip_reduce(torch, hip, dtype, "sum", ins, in_offsets=in_offs, out_offsets=[off])
            H.assert_bits_equal(got, want, "%s count=%d off=%d" % (dtype, count, off))


@pytest.mark.parametrize("n_out", [1, 2, 3, 8])
def test_multi_output(hip, oracle, n_out):
    import torch
    count = 100003
    for dtype in ("bf16", "f16", "f32"):
        ins = _inputs(dtype, "sum", 4, count, seed=11)
        want = oracle.reduce(dtype, "sum", ins)
        outs = H.hip_reduce(torch, hip, dtype, "sum", ins, n_out=n_out,
                            out_offsets=[(2 * j * H.ELEM_BYTES[dtype]) % 64 for j in range(n_out)])
        for j, got in enumerate(outs):
            H.assert_bits_equal(got, want, "%s out %d of %d" % (dtype, j, n_out))


def test_in_place_ring_step(hip, oracle):
    """Output 0 is also input 1 (the in-place form a ring step uses)."""
    import torch
    count = 300007
    a = H.gen("bf16", count, 21, 0)
    b = H.gen("bf16", count, 21, 1)
    want = oracle.reduce("bf16", "sum", [a, b])
    d_a = H.DevBuf(torch, "bf16", count, 6, src=a)
    d_b = H.DevBuf(torch, "bf16", count, 10, src=b)
    d_send = H.DevBuf(torch, "bf16", count, 0)
    hip.reduce_copy("bf16", "sum", [d_a.ptr, d_b.ptr], [d_b.ptr, d_send.ptr], count,
                    torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    H.assert_bits_equal(d_b.download(), want, "in-place output")
    H.assert_bits_equal(d_send.download(), want, "send buffer")
    H.assert_bits_equal(d_a.download(), a, "input untouched")
    assert d_b.guards_intact() and d_send.guards_intact()


def test_fold_order_is_input_order(hip, oracle):
    """f32 inputs with a wide exponent spread: folding the same buffers in reversed order gives
    different bits, and the kernel matches the checker for both orders (sum and prod)."""
    import torch
    count = 50021
    for n_in in (3, 8):
        ins = []
        for k in range(n_in):
            mag = np.exp2(oracle.fill_uniform_f32(count, 300, 10 + k, -20.0, 20.0)).astype(np.float32)
            ins.append(oracle.fill_uniform_f32(count, 300, k, -1.0, 1.0) * mag)
        fwd, rev = oracle.reduce("f32", "sum", ins), oracle.reduce("f32", "sum", ins[::-1])
        assert not np.array_equal(fwd.view(np.uint32), rev.view(np.uint32)), "input not order-sensitive: weak test"
        (got,) = H.hip_reduce(torch, hip, "f32", "sum", ins)
        H.assert_bits_equal(got, fwd, "forward order n_in=%d" % n_in)
        (got,) = H.hip_reduce(torch, hip, "f32", "sum", ins[::-1])
        H.assert_bits_equal(got, rev, "reversed order n_in=%d" % n_in)
    # (1e8 + 1) - 1e8 = 0 from the left, 1 when the big terms cancel first
    a, b, c = (np.full(1000, v, dtype=np.float32) for v in (1e8, 1.0, -1e8))
    (got,) = H.hip_reduce(torch, hip, "f32", "sum", [a, b, c])
    assert np.all(got == 0.0)
    (got,) = H.hip_reduce(torch, hip, "f32", "sum", [a, c, b])
    assert np.all(got == 1.0)


def test_special_values(hip, oracle):
    """inf, NaN, signed zero, subnormals and rounding ties through the bf16 / f16 / f32 paths."""
    import torch
    f = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-40, -1e-40, 3.0e38, -3.0e38, 65504.0,
                  65520.0, 1.00390625, 1.01171875, 5.9604645e-8, 2.98e-8, 6.1e-5, 1e-45], dtype=np.float32)
    pairs = np.array(list(itertools.product(f, f)), dtype=np.float32)
    for dtype in ("f32", "bf16", "f16"):
        x = pairs[:, 0].copy() if dtype == "f32" else oracle.narrow(dtype, pairs[:, 0])
        y = pairs[:, 1].copy() if dtype == "f32" else oracle.narrow(dtype, pairs[:, 1])
        for compute in ("sum", "prod", "min", "max"):
            want = oracle.reduce(dtype, compute, [x, y])
            (got,) = H.hip_reduce(torch, hip, dtype, compute, [x, y])
            if dtype == "f32":
                wn, gn = np.isnan(want), np.isnan(got)
            else:
                wn, gn = np.isnan(oracle.widen(dtype, want)), np.isnan(oracle.widen(dtype, got))
            assert np.array_equal(wn, gn), "%s %s: NaN positions differ" % (dtype, compute)
            H.assert_bits_equal(np.where(wn, 0, H.bits(got)), np.where(wn, 0, H.bits(want)),
                                "%s %s specials" % (dtype, compute))


def _nan_inputs(oracle, dtype, n, seed):
    """Three inputs of n elements; by element index modulo 8: 0 no NaN, 1-3 exactly one NaN (first, middle,
    last input; random sign and payload, quiet or signalling), 4 a signalling NaN alone, 5 two NaNs
    (first and last input), 6 +inf / -inf / finite, 7 zero / inf / finite."""
    rng = np.random.default_rng(seed)
    f = [rng.uniform(0.5, 2.0, n).astype(np.float32) for _ in range(3)]
    cat = np.arange(n) % 8

    def nans(quiet=None):
        sign = rng.integers(0, 2, n).astype(np.uint32) << 31
        q = (rng.integers(0, 2, n).astype(np.uint32) if quiet is None else np.full(n, quiet, np.uint32)) << 22
        return (sign | np.uint32(0x7f800000) | q | rng.integers(1 << 14, 1 << 22, n).astype(np.uint32)).view(np.float32)

    for k, c in ((0, 1), (1, 2), (2, 3)):
        f[k] = np.where(cat == c, nans(), f[k])
    f[1] = np.where(cat == 4, nans(0), f[1])
    f[0] = np.where(cat == 5, nans(), f[0])
    f[2] = np.where(cat == 5, nans(), f[2])
    f[0] = np.where(cat == 6, np.float32(np.inf), np.where(cat == 7, np.float32(0.0), f[0]))
    f[1] = np.where(cat == 6, np.float32(-np.inf), np.where(cat == 7, np.float32(np.inf), f[1]))

    def store(x):
        u = x.view(np.uint32)
        if dtype == "f32":
            return x.copy()
        if dtype == "f64":   # NaN payload and sign placed by hand (a cast would be free to change them)
            with np.errstate(invalid="ignore"):
                d = x.astype(np.float64).view(np.uint64)
            isn = (u & 0x7fffffff) > 0x7f800000
            hand = ((u.astype(np.uint64) >> np.uint64(31)) << np.uint64(63)) | np.uint64(0x7ff0000000000000) | ((u.astype(np.uint64) & np.uint64(0x7fffff)) << np.uint64(29))
            return np.where(isn, hand, d).view(np.float64)
        if dtype == "bf16":
            return np.where((u & 0x7fffffff) > 0x7f800000, u >> 16, oracle.narrow("bf16", x).astype(np.uint32)).astype(np.uint16)
        hn = ((u >> 16) & 0x8000) | 0x7c00 | ((u >> 13) & 0x3ff)
        return np.where((u & 0x7fffffff) > 0x7f800000, hn, oracle.narrow("f16", x).astype(np.uint32)).astype(np.uint16)

    return [store(x) for x in f], cat


def _check_nan_bits(oracle, dtype, compute, ins, cat, got, what):
    """Bit for bit against the CPU checker, NaNs included (sign, payload, quiet bit).  One exception, which
    the semantics leave open: a sum or product of SEVERAL NaN inputs is a quiet NaN carrying the sign and
    payload of one of them (x86 keeps the first operand's, the GPU's instruction whichever the compiler put
    first); there the result must be one of the candidates."""
    want = oracle.reduce(dtype, compute, ins)
    wb, gb = H.bits(want), H.bits(got)
    several = (cat == 5) & (compute in ("sum", "prod"))
    H.assert_bits_equal(np.where(several, 0, gb), np.where(several, 0, wb), what)
    if several.any():
        zero = np.zeros_like(ins[1])
        cand = [H.bits(oracle.reduce(dtype, "sum", [ins[k], zero])) for k in (0, 2)]   # the NaN of input k, quieted
        ok = (gb == cand[0]) | (gb == cand[1])
        assert ok[several].all(), "%s: a several-NaN result is none of its inputs' NaNs" % what
    # every NaN that comes out of arithmetic is quiet
    if compute in ("sum", "prod"):
        quiet = {"f32": 1 << 22, "f64": 1 << 51, "bf16": 1 << 6, "f16": 1 << 9}[dtype]
        isn = np.isnan(got) if dtype in ("f32", "f64") else np.isnan(oracle.widen(dtype, got))
        assert ((gb[isn] & np.asarray(quiet, dtype=gb.dtype)) != 0).all(), "%s: a signalling NaN came out" % what


def test_nan_results_bit_for_bit(hip, oracle):
    """NaN sign, payload and quiet bit through packs, head / tail elements and queue parts."""
    import torch
    n = 8 * 1031 + 5
    stream = torch.cuda.current_stream().cuda_stream
    for dtype in ("f32", "bf16", "f16", "f64"):
        es = H.ELEM_BYTES[dtype]
        ins, cat = _nan_inputs(oracle, dtype, n, 17)
        for compute in ("sum", "prod", "min", "max"):
            for offs in ([0, 0, 0], [es, 3 * es, 0]):
                (got,) = H.hip_reduce(torch, hip, dtype, compute, ins, in_offsets=offs, out_offsets=[offs[0]])
                _check_nan_bits(oracle, dtype, compute, ins, cat, got, "%s %s direct, offsets %s" % (dtype, compute, offs))
            d_in = [H.DevBuf(torch, dtype, n, es * k, src=a) for k, a in enumerate(ins)]
            d_out = H.DevBuf(torch, dtype, n, es)
            g = hip.Graph([dict(dtype=dtype, compute=compute, ins=[b.ptr for b in d_in], outs=[d_out.ptr], count=n)], 8192)
            g.run(stream)
            assert g.status(stream) == (1, 1)
            _check_nan_bits(oracle, dtype, compute, ins, cat, d_out.download(), "%s %s through the queue" % (dtype, compute))
            g.destroy()


def test_argument_errors(hip):
    import torch
    t = torch.zeros(1024, dtype=torch.float32, device="cuda")
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy(99, "sum", [t], [t], 4)
    assert e.value.code == hip.ERR_UNSUPPORTED
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", 7, [t, t], [t], 4)
    assert e.value.code == hip.ERR_UNSUPPORTED
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", "sum", [t] * 9, [t], 4)
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", "sum", [t], [], 4)
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", "sum", [t], [t], -1)
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", "sum", [t.data_ptr() + 2], [t], 4)
    assert e.value.code == hip.ERR_MISALIGNED
    with pytest.raises(hip.PcclError) as e:
        hip.reduce_copy("f32", "sum", [0], [t], 4)
    assert e.value.code == hip.ERR_INVALID_ARG
    hip.reduce_copy("f32", "sum", [t], [t], 0)  # empty op is a no-op
    torch.cuda.synchronize()


def test_every_kernel_variant_through_the_knobs(hip, oracle):
    """The launch policy picks cache treatment, kernel shape and occupancy cap from operand sizes
    that only large runs reach; the tuning knobs force each variant on small ragged inputs:
    cache treatment 0 (cacheable) / 1 (non-temporal) / 2 (non-temporal loads, write-through
    stores) x lean / 1 pack per lane / 4 packs per lane x full grid / persistent grid."""
    import torch
    cases = [("bf16", 8, 1, 256 * 8 * 5, 0), ("bf16", 3, 2, 70001, 2), ("f8e4m3", 1, 8, 93744, 1), ("f32", 2, 8, 50001, 4), ("f32", 2, 1, 4099, 4), ("f32", 2, 3, 1 << 16, 0),
             ("i32", 4, 1, 131071, 12), ("f16", 1, 2, 50001, 6), ("f8e4m3", 5, 1, 30011, 3), ("bf16", 1, 1, 1 << 17, 0)]
    try:
        for dtype, n_in, n_out, count, off in cases:
            ins = _inputs(dtype, "sum", n_in, count, seed=300 + n_in)
            want = oracle.reduce(dtype, "sum", ins)
            offs_in = [(off * (k + 1)) % 64 for k in range(n_in)]
            offs_out = [(off * (k + 2)) % 64 for k in range(n_out)]
            for mem in (0, 1, 2):
                for unroll in (0, 1, 4):
                    for wg in (0, 2):
                        hip.set_tuning(wg, mem)
                        hip.set_unroll(unroll)
                        hip.set_occupancy_lds(65536 if wg == 0 else 0)
                        got = H.hip_reduce(torch, hip, dtype, "sum", ins, n_out=n_out, in_offsets=offs_in,
                                           out_offsets=offs_out)
                        for g in got:
                            H.assert_bits_equal(g, want, "%s %d->%d count=%d mem=%d unroll=%d wg=%d"
                                                % (dtype, n_in, n_out, count, mem, unroll, wg))
    finally:
        hip.set_tuning(0, -1)
        hip.set_unroll(-1)
        hip.set_occupancy_lds(-1)


def test_operands_longer_than_one_launch_covers(hip, oracle):
    """Operands beyond what a launch's grid can cover (32 GiB by default) run as several launches over
    consecutive slices.  With the slice set to 64 KiB and 4 KiB: ragged counts, operands off the 16-byte
    grid, reduce-copy and accumulate, against the checker; and the setter's argument checks."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    try:
        for slice_bytes in (65536, 4096):
            hip.set_slice_bytes(slice_bytes)
            for dtype, compute, n_in, n_out, count, off in (("bf16", "sum", 8, 1, 100003, 0), ("f32", "max", 2, 2, 70001, 4),
                                                            ("f8e4m3", "sum", 3, 1, 300001, 3), ("i32", "sum", 1, 3, 65537, 12),
                                                            ("f64", "prod", 2, 1, 8192 * 3, 0), ("f16", "min", 4, 2, 32768, 2)):
                es = H.ELEM_BYTES[dtype]
                off = off // es * es
                kw = dict(kind="uniform", lo=0.5, hi=2.0) if compute == "prod" else {}
                ins = [H.gen(dtype, count, 410 + n_in, k, **kw) for k in range(n_in)]
                want = oracle.reduce(dtype, compute, ins)
                got = H.hip_reduce(torch, hip, dtype, compute, ins, n_out=n_out, in_offsets=[(off * (k + 1)) % 64 for k in range(n_in)],
                                   out_offsets=[(off * (k + 2)) % 64 for k in range(n_out)])
                for g in got:
                    H.assert_bits_equal(g, want, "%s %s %d->%d count=%d slice=%d" % (dtype, compute, n_in, n_out, count, slice_bytes))
                # accumulate: the first input folded into copies of the others
                dsts = [H.DevBuf(torch, dtype, count, (off * (j + 1)) % 64, src=ins[min(j + 1, n_in - 1)]) for j in range(n_out)]
                src = H.DevBuf(torch, dtype, count, off, src=ins[0])
                hip.accumulate(dtype, compute, src.ptr, [d.ptr for d in dsts], count, stream)
                torch.cuda.synchronize()
                for j, d in enumerate(dsts):
                    H.assert_bits_equal(d.download(), oracle.reduce(dtype, compute, [ins[min(j + 1, n_in - 1)], ins[0]]),
                                        "accumulate %s %s count=%d slice=%d" % (dtype, compute, count, slice_bytes))
                    assert d.guards_intact()
        for bad in (100, 4097, -4096, (32 << 30) + 4096):
            with pytest.raises(hip.PcclError) as e:
                hip.set_slice_bytes(bad)
            assert e.value.code == hip.ERR_INVALID_ARG
    finally:
        hip.set_slice_bytes(0)


# ---- the fold rounds to binary32 at every step, then once to the element type ----------------

def _tie_tuples(oracle, dtype, compute, n_in, want, seed):
    """Tuples of n_in elements whose binary32 left fold lies EXACTLY between two values of the
    element type.  There, rounding the last step's exact result straight to the element type
    (what a fused multiply-and-narrow instruction does) differs from rounding it to binary32
    first in about half the cases, so these are the inputs that tell the two apart."""
    rng = np.random.default_rng(seed)
    low_bits = 13 if dtype == "f16" else 16
    found = []
    while sum(len(f) for f in found) < want:
        vals = rng.uniform(0.5, 2.0, (1 << 20, n_in)).astype(np.float32)
        if compute == "sum":
            vals *= rng.choice(np.float32([1, -1, 0.25, 8]), vals.shape)
        bits = oracle.narrow(dtype, vals)
        x = oracle.widen(dtype, bits)
        acc = x[:, 0].copy()
        for k in range(1, n_in):
            acc = (acc * x[:, k] if compute == "prod" else acc + x[:, k]).astype(np.float32)
        tie = (acc.view(np.uint32) & np.uint32((1 << low_bits) - 1)) == np.uint32(1 << (low_bits - 1))
        found.append(bits[tie])
    return np.concatenate(found)[:want]


@pytest.mark.parametrize("dtype", ["f16", "bf16"])
def test_fold_rounds_to_binary32_before_narrowing(hip, oracle, dtype):
    """Every path an element can take (16-byte packs, the element-wise head and tail of an
    unaligned buffer, parts of the queue executor) must round like the CPU checker on inputs
    whose binary32 fold is a tie of the element type."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    for compute, n_in in (("prod", 8), ("prod", 3), ("sum", 4), ("sum", 8)):
        ties = _tie_tuples(oracle, dtype, compute, n_in, 7 * 40, 4242 + n_in)
        ins = [np.ascontiguousarray(ties[:, k]) for k in range(n_in)]
        want = oracle.reduce(dtype, compute, ins)
        what = "%s %s %d inputs" % (dtype, compute, n_in)
        # all through packs (aligned), and with an element-wise head and tail (offset buffers)
        H.assert_bits_equal(H.hip_reduce(torch, hip, dtype, compute, ins)[0], want, what + ", aligned")
        got = H.hip_reduce(torch, hip, dtype, compute, ins, in_offsets=[2 * (k + 1) for k in range(n_in)], out_offsets=[6])[0]
        H.assert_bits_equal(got, want, what + ", offset buffers")
        # seven elements at a time: every element goes the element-wise way
        for lo in range(0, len(want), 7):
            got = H.hip_reduce(torch, hip, dtype, compute, [a[lo:lo + 7] for a in ins], out_offsets=[2])[0]
            H.assert_bits_equal(got, want[lo:lo + 7], what + ", elements %d.." % lo)
        # the queue executor, parts of 1 KiB starting off 16 bytes
        d_in = [H.DevBuf(torch, dtype, len(want), 2 * (k % 5), src=a) for k, a in enumerate(ins)]
        d_out = H.DevBuf(torch, dtype, len(want), 10)
        g = hip.Graph([dict(dtype=dtype, compute=compute, ins=[b.ptr for b in d_in], outs=[d_out.ptr], count=len(want))],
                      tile_bytes=1024)
        g.run(stream)
        assert g.status(stream) == (1, 1)
        H.assert_bits_equal(d_out.download(), want, what + ", queue")
        g.destroy()
