"""GPU parity of the 8-bit float dtypes (OCP E4M3FN and E5M2) through the C ABI: every pair of
encodings under every compute (which exercises the hardware widening of all 256 codes and the
narrowing on every tie the format has), ragged counts at every byte offset, multi-input folds,
the queue executor and the accumulate entry point."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

F8 = ("f8e4m3", "f8e5m2")


def _nan_mask(oracle, dtype, a):
    return np.isnan(oracle.widen(dtype, a))


def _assert_f8_equal(oracle, dtype, got, want, what):
    """Bit-exact outside NaN; NaN positions must agree (any NaN encoding of the format)."""
    gn, wn = _nan_mask(oracle, dtype, got), _nan_mask(oracle, dtype, want)
    assert np.array_equal(gn, wn), "%s: NaN positions differ" % what
    H.assert_bits_equal(np.where(wn, 0, got), np.where(wn, 0, want), what)


@pytest.mark.parametrize("dtype", F8)
@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_every_pair_of_encodings(hip, oracle, dtype, compute):
    import torch
    codes = np.arange(256, dtype=np.uint8)
    x, y = np.repeat(codes, 256), np.tile(codes, 256)
    want = oracle.reduce(dtype, compute, [x, y])
    (got,) = H.hip_reduce(torch, hip, dtype, compute, [x, y])
    _assert_f8_equal(oracle, dtype, got, want, "%s %s all pairs" % (dtype, compute))


@pytest.mark.parametrize("dtype", F8)
@pytest.mark.parametrize("compute", ["sum", "prod"])
def test_random_encodings_every_nin(hip, oracle, dtype, compute):
    """Uniformly random bytes: most folds overflow, so every instantiation shows that it saturates."""
    import torch
    rng = np.random.default_rng(22)
    for n_in in range(2, 9):
        for count, off in ((70001, 1), (1 << 18, 0)):
            ins = [rng.integers(0, 256, size=count, dtype=np.uint64).astype(np.uint8) for _ in range(n_in)]
            want = oracle.reduce(dtype, compute, ins)
            (got,) = H.hip_reduce(torch, hip, dtype, compute, ins, in_offsets=[off] * n_in, out_offsets=[off])
            _assert_f8_equal(oracle, dtype, got, want, "%s %s n_in=%d count=%d" % (dtype, compute, n_in, count))


@pytest.mark.parametrize("dtype", F8)
def test_three_input_sums_hit_rounding_cases(hip, oracle, dtype):
    """Sums of three values carry more low bits than a pair can; random finite triples."""
    import torch
    rng = np.random.default_rng(21)
    ins = [rng.integers(0, 256, size=1 << 20, dtype=np.uint64).astype(np.uint8) for _ in range(3)]
    want = oracle.reduce(dtype, "sum", ins)
    (got,) = H.hip_reduce(torch, hip, dtype, "sum", ins)
    _assert_f8_equal(oracle, dtype, got, want, dtype)


@pytest.mark.parametrize("dtype", F8)
@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_all_nin_ragged(hip, oracle, dtype, compute):
    import torch
    for n_in in range(1, 9):
        for count in (1, 5, 257, 4099, 70001):
            if compute == "prod":
                ins = [H.gen(dtype, count, 30 + n_in, k, kind="uniform", lo=0.5, hi=2.0) for k in range(n_in)]
            else:
                ins = [H.gen(dtype, count, 30 + n_in, k, kind="normal") for k in range(n_in)]
            want = oracle.reduce(dtype, compute, ins)
            (got,) = H.hip_reduce(torch, hip, dtype, compute, ins)
            H.assert_bits_equal(got, want, "%s %s n_in=%d count=%d" % (dtype, compute, n_in, count))


def test_every_byte_offset(hip, oracle):
    import torch
    dtype = "f8e4m3"
    for count in (1, 3, 15, 16, 17, 63, 64, 65, 255, 4097, 20001):
        ins = [H.gen(dtype, count, 8, k) for k in range(3)]
        want = oracle.reduce(dtype, "sum", ins)
        for off in range(0, 32):
            in_offs = [(off + 5 * k) % 32 for k in range(3)]
            got = H.hip_reduce(torch, hip, dtype, "sum", ins, n_out=2, in_offsets=in_offs,
                               out_offsets=[off, (off * 7 + 3) % 32])
            for g in got:
                H.assert_bits_equal(g, want, "count=%d off=%d" % (count, off))


@pytest.mark.parametrize("dtype", F8)
def test_large_aligned_takes_the_streaming_path(hip, oracle, dtype):
    """64 MiB per operand, 4 inputs, 2 outputs: the lean kernel with streaming hints."""
    import torch
    n = 64 << 20
    ins = [H.gen(dtype, n, 40, k, sigma=100.0) for k in range(4)]   # wide enough to saturate often
    want = np.empty_like(ins[0])
    oracle.reduce_copy(dtype, "sum", ins, [want], nthreads=8)
    got = H.hip_reduce(torch, hip, dtype, "sum", ins, n_out=2)
    for g in got:
        H.assert_bits_equal(g, want, dtype)


@pytest.mark.parametrize("dtype", F8)
def test_queue_executor(hip, oracle, dtype):
    """A chain through the queue: t = a + b + c; u = t + d; v = copy of u."""
    import torch
    n = 300_001
    a, b, c, d = (H.gen(dtype, n, 50, k, sigma=150.0) for k in range(4))
    bufs = [H.DevBuf(torch, dtype, n, src=x) for x in (a, b, c, d)]
    t, u, v = (H.DevBuf(torch, dtype, n) for _ in range(3))
    ops = [dict(dtype=dtype, compute="sum", ins=[bufs[0].ptr, bufs[1].ptr, bufs[2].ptr], outs=[t.ptr], count=n),
           dict(dtype=dtype, compute="sum", ins=[t.ptr, bufs[3].ptr], outs=[u.ptr], count=n, deps=[0]),
           dict(dtype=dtype, compute="sum", ins=[u.ptr], outs=[v.ptr], count=n, deps=[1])]
    g = hip.Graph(ops, tile_bytes=16384)
    g.run(torch.cuda.current_stream().cuda_stream)
    assert g.status(torch.cuda.current_stream().cuda_stream) == (3, 3)
    want_t = oracle.reduce(dtype, "sum", [a, b, c])
    want_u = oracle.reduce(dtype, "sum", [want_t, d])
    H.assert_bits_equal(t.download(), want_t, "t")
    H.assert_bits_equal(u.download(), want_u, "u")
    H.assert_bits_equal(v.download(), want_u, "v")
    for x in (t, u, v):
        assert x.guards_intact()
    g.destroy()


@pytest.mark.parametrize("dtype", F8)
def test_accumulate(hip, oracle, dtype):
    import torch
    n = 100_003
    src = H.gen(dtype, n, 60, 0, sigma=300.0)
    dst0 = [H.gen(dtype, n, 60, 1 + k, sigma=300.0) for k in range(3)]
    d_src = H.DevBuf(torch, dtype, n, src=src, offset=3)
    d_dst = [H.DevBuf(torch, dtype, n, src=x, offset=k) for k, x in enumerate(dst0)]
    hip.accumulate(dtype, "sum", d_src.ptr, [x.ptr for x in d_dst], n, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    for k, x in enumerate(d_dst):
        H.assert_bits_equal(x.download(), oracle.reduce(dtype, "sum", [dst0[k], src]), "dst %d" % k)
        assert x.guards_intact()
