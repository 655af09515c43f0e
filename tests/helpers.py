"""Shared helpers of the parity tests: seeded inputs from the CPU checker's generator,
device staging with chosen misalignment, and bit-level comparison."""
import numpy as np

import pccl_oracle as orc

ELEM_BYTES = {"f32": 4, "i32": 4, "bf16": 2, "f16": 2, "f8e4m3": 1, "f8e5m2": 1, "f64": 8, "u32": 4}
STORAGE = {"f32": np.float32, "i32": np.int32, "bf16": np.uint16, "f16": np.uint16,
           "f8e4m3": np.uint8, "f8e5m2": np.uint8, "f64": np.float64, "u32": np.uint32}


def gen(dtype, count, seed, stream, kind="normal", **kw):
    """One seeded input buffer in its storage type."""
    if dtype == "i32":
        return orc.fill_int32(count, seed, stream, kw.get("lo", -(1 << 20)), kw.get("hi", 1 << 20))
    if dtype == "u32":
        # the whole range by default, so that values above 2^31 tell unsigned min / max from signed
        lo, hi = kw.get("lo", 0), kw.get("hi", (1 << 32) - 1)
        return orc.fill_int32(count, seed, stream, lo - (1 << 31), hi - (1 << 31)).view(np.uint32) ^ np.uint32(1 << 31)
    if kind == "uniform":
        a = orc.fill_uniform_f32(count, seed, stream, kw.get("lo", -1.0), kw.get("hi", 1.0))
        if dtype == "f64":  # a second draw fills the mantissa bits a binary32 does not have
            b = orc.fill_uniform_f32(count, seed, stream + 1000, 0.0, 1.0)
            return a.astype(np.float64) * (1.0 + b.astype(np.float64) * 2.0 ** -24)
        return a if dtype == "f32" else orc.narrow(dtype, a)
    return orc.fill_normal(dtype, count, seed, stream, kw.get("mean", 0.0), kw.get("sigma", 1.0))


def bits(a):
    """Bit pattern view for exact comparison (NaN-safe)."""
    a = np.ascontiguousarray(a)
    if a.dtype == np.float32:
        return a.view(np.uint32)
    if a.dtype == np.int32:
        return a.view(np.uint32)
    if a.dtype == np.float64:
        return a.view(np.uint64)
    return a


def assert_bits_equal(got, want, what=""):
    g, w = bits(got), bits(want)
    assert g.shape == w.shape, "%s: shape %s vs %s" % (what, g.shape, w.shape)
    if not np.array_equal(g, w):
        bad = np.flatnonzero(g != w)
        i = int(bad[0])
        raise AssertionError("%s: %d of %d elements differ, first at %d: got 0x%x want 0x%x"
                             % (what, bad.size, g.size, i, int(g[i]), int(w[i])))


class DevBuf:
    """A device buffer holding `count` elements at `offset` bytes past a 256-byte boundary."""

    def __init__(self, torch, dtype, count, offset=0, src=None, fill=0xFF):
        self.dtype, self.count, self.offset = dtype, count, offset
        self.nbytes = count * ELEM_BYTES[dtype]
        # torch allocations are at least 256-byte aligned; keep a guard band on both sides
        self.guard = 256
        self.raw = torch.full((self.guard + offset + self.nbytes + self.guard,), fill, dtype=torch.uint8,
                              device="cuda")
        assert self.raw.data_ptr() % 256 == 0
        self.ptr = self.raw.data_ptr() + self.guard + offset
        self._torch = torch
        if src is not None:
            self.upload(src)

    def view(self):
        lo = self.guard + self.offset
        return self.raw[lo:lo + self.nbytes]

    def upload(self, a):
        a = np.ascontiguousarray(a)
        assert a.nbytes == self.nbytes
        self.view().copy_(self._torch.from_numpy(a.view(np.uint8).reshape(-1)))

    def download(self):
        return self.view().cpu().numpy().view(STORAGE[self.dtype]).copy()

    def guards_intact(self, fill=0xFF):
        lo = self.guard + self.offset
        head = self.raw[:lo].cpu().numpy()
        tail = self.raw[lo + self.nbytes:].cpu().numpy()
        return bool((head == fill).all() and (tail == fill).all())


def hip_reduce(torch, hip, dtype, compute, ins_np, n_out=1, in_offsets=None, out_offsets=None, count=None):
    """Uploads, runs one pccl_hip_reduce_copy through the C ABI, downloads all outputs."""
    count = ins_np[0].size if count is None else count
    in_offsets = in_offsets or [0] * len(ins_np)
    out_offsets = out_offsets or [0] * n_out
    d_in = [DevBuf(torch, dtype, count, off, src=a[:count]) for a, off in zip(ins_np, in_offsets)]
    d_out = [DevBuf(torch, dtype, count, off) for off in out_offsets]
    stream = torch.cuda.current_stream().cuda_stream
    hip.reduce_copy(dtype, compute, [b.ptr for b in d_in], [b.ptr for b in d_out], count, stream)
    torch.cuda.synchronize()
    outs = [b.download() for b in d_out]
    for b in d_out:
        assert b.guards_intact(), "kernel wrote outside its output buffer"
    return outs
