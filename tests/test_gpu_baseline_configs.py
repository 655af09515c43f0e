"""GPU parity at the full sizes of the five baseline configurations.  Inputs are the CPU checker's
seeded inputs (its splitmix64 counter generator, evaluated on the device and pinned against the host
form), downloaded once, and the CPU checker (threaded form, same arithmetic as the scalar form)
computes the expected bytes; every comparison is bit-exact."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

THREADS = 16
NPDT = {"f32": np.float32, "i32": np.int32, "bf16": np.uint16, "f16": np.uint16}


def _stream(torch):
    return torch.cuda.current_stream().cuda_stream


_M64 = (1 << 64) - 1
_GOLD = 0x9e3779b97f4a7c15


def _s64(v):
    """A 64-bit pattern as the signed value torch's int64 holds."""
    v &= _M64
    return v - (1 << 64) if v >> 63 else v


def _mix64_int(z):
    z &= _M64
    z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & _M64
    z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & _M64
    return z ^ (z >> 31)


def _mix64_dev(z):
    """splitmix64's finaliser on an int64 tensor: products wrap, shifts are made logical."""
    lsr = lambda x, k: (x >> k) & ((1 << (64 - k)) - 1)
    z = (z ^ lsr(z, 30)) * _s64(0xbf58476d1ce4e5b9)
    z = (z ^ lsr(z, 27)) * _s64(0x94d049bb133111eb)
    return z ^ lsr(z, 31)


def _dev_random(torch, dtype, count, seed, kind="normal", sigma=1.0, lo=0.5, hi=2.0, stream=0):
    """Seeded input generated ON the device by the CPU checker's own counter generator
    (oracle/pccl_oracle.c: rng_u64 = splitmix64 finaliser over (seed, stream, index); fill_int32,
    fill_uniform_f32, then the type's round-to-nearest-even narrowing), so that the full-size inputs are
    those of H.gen(dtype, count, seed, stream, kind="uniform", ...) bit for bit without a host
    pass over gigabytes (test_device_generator_is_the_host_generator checks windows of it).
    kind "normal" asks for zero mean and the given sigma: uniform in [-sigma * sqrt 3, sigma * sqrt 3)."""
    key = _mix64_int(seed * _GOLD + stream + 0x632be59bd9b4e019)
    if kind == "normal":
        lo, hi = -sigma * 1.7320508, sigma * 1.7320508
    tdt = {"f32": torch.float32, "bf16": torch.bfloat16, "f16": torch.float16, "i32": torch.int32}[dtype]
    out = torch.empty(count, dtype=tdt, device="cuda")
    step = 1 << 25
    for a in range(0, count, step):
        b = min(count, a + step)
        idx = torch.arange(a + 1, b + 1, dtype=torch.int64, device="cuda")
        x = _mix64_dev(idx * _s64(_GOLD) + _s64(key))
        if dtype == "i32":
            span = (1 << 21) + 1          # values in [-2^20, 2^20]
            hi32, lo32 = (x >> 32) & 0xffffffff, x & 0xffffffff
            out[a:b] = ((hi32 * ((1 << 32) % span) + lo32) % span - (1 << 20)).to(torch.int32)   # x mod span, x unsigned
        else:
            u = ((x >> 40) & 0xffffff).to(torch.float32) * (1.0 / 16777216.0)
            lo32f, d32f = np.float32(lo), np.float32(np.float32(hi) - np.float32(lo))
            v = u * float(d32f)          # two roundings, as the checker's lo + (hi - lo) * u without contraction
            v = v + float(lo32f)
            out[a:b] = v.to(tdt)
    return out


def _host(t, dtype):
    """Device tensor -> numpy array in the checker's storage type."""
    a = t.cpu()
    if dtype in ("bf16", "f16"):
        return a.view(__import__("torch").int16).numpy().view(np.uint16)
    return a.numpy()


def _expect(oracle, dtype, compute, host_ins):
    out = np.empty_like(host_ins[0])
    oracle.reduce_copy(dtype, compute, host_ins, [out], nthreads=THREADS)
    return out


def test_device_generator_is_the_host_generator(hip, oracle):
    """The inputs of the full-size tests are the CPU checker's seeded inputs: windows at the start, across
    a chunk boundary of the device loop and at the end agree bit for bit, for every dtype used."""
    import torch
    count = (1 << 25) + 4099
    windows = [slice(0, 1 << 16), slice((1 << 25) - 999, (1 << 25) + 999), slice(count - 4099, count)]
    for dtype, kw, host_kw in (("i32", {}, dict(lo=-(1 << 20), hi=1 << 20)),
                               ("f32", dict(kind="uniform", lo=0.5, hi=2.0), dict(kind="uniform", lo=0.5, hi=2.0)),
                               ("bf16", dict(sigma=1e-2), dict(kind="uniform", lo=-1e-2 * 1.7320508, hi=1e-2 * 1.7320508)),
                               ("f16", dict(kind="uniform", lo=-2.0, hi=2.0), dict(kind="uniform", lo=-2.0, hi=2.0))):
        dev = _host(_dev_random(torch, dtype, count, 77, stream=3, **kw), dtype)
        want = H.gen(dtype, count, 77, 3, **host_kw)
        for w in windows:
            H.assert_bits_equal(dev[w], want[w], "%s window %s" % (dtype, w))


def test_config2_ring_rank_share_full_size(hip, oracle):
    """bf16 ring all-reduce, one rank's share at world 8: 256 MiB gradient = 8 x 32 MiB chunks, 7
    reduce-copy steps (peer chunk + local chunk -> output chunk + send buffer) and 7 copy steps."""
    import torch
    W, ce = 8, 1 << 24
    grad = _dev_random(torch, "bf16", W * ce, 1, sigma=1e-2)
    peers = [_dev_random(torch, "bf16", ce, 100 + s, sigma=1e-2) for s in range(W - 1)]
    result = torch.zeros(W * ce, dtype=torch.bfloat16, device="cuda")
    send = torch.zeros(ce, dtype=torch.bfloat16, device="cuda")
    h_grad, h_peers = _host(grad, "bf16"), [_host(p, "bf16") for p in peers]
    h_result = np.zeros(W * ce, dtype=np.uint16)
    for s in range(W - 1):
        c = (W - 1 - s) % W
        sl = slice(c * ce, (c + 1) * ce)
        hip.reduce_copy("bf16", "sum", [peers[s], grad[sl]], [result[sl], send], ce, _stream(torch))
        torch.cuda.synchronize()
        want = _expect(oracle, "bf16", "sum", [h_peers[s], h_grad[sl]])
        h_result[sl] = want
        H.assert_bits_equal(_host(send, "bf16"), want, "send buffer after reduce step %d" % s)
    for s in range(W - 1):
        c = (W - s) % W
        sl = slice(c * ce, (c + 1) * ce)
        hip.reduce_copy("bf16", "sum", [peers[s]], [result[sl]], ce, _stream(torch))
        h_result[sl] = h_peers[s]
    torch.cuda.synchronize()
    H.assert_bits_equal(_host(result, "bf16"), h_result, "assembled 256 MiB result")


@pytest.mark.parametrize("dtype, n_out, count", [("bf16", 1, 1 << 26), ("f16", 2, 1 << 26), ("bf16", 1, 1 << 27)])
def test_config3_eight_input_reduce_full_size(hip, oracle, dtype, n_out, count):
    """8 inputs -> 1 (or 2) outputs, 128 MiB and 256 MiB per buffer, fixed input order."""
    import torch
    ins = [_dev_random(torch, dtype, count, 2000 + k) for k in range(8)]
    outs = [torch.zeros(count, dtype=ins[0].dtype, device="cuda") for _ in range(n_out)]
    hip.reduce_copy(dtype, "sum", ins, outs, count, _stream(torch))
    torch.cuda.synchronize()
    want = _expect(oracle, dtype, "sum", [_host(t, dtype) for t in ins])
    for j, o in enumerate(outs):
        H.assert_bits_equal(_host(o, dtype), want, "%s 8->%d output %d" % (dtype, n_out, j))
    # the same fold in torch (fp32 accumulate, input order, one rounding) as a second opinion
    acc = ins[0][:1 << 22].float()
    for k in range(1, 8):
        acc = acc + ins[k][:1 << 22].float()
    assert torch.equal(acc.to(ins[0].dtype), outs[0][:1 << 22])


def _normal_on_device(torch, oracle, dtype, count, seed, stream, sigma):
    """True N(0, sigma) input from the CPU checker's Box-Muller generator (threaded on the host, uploaded): the
    values the configurations name, tails included, where _dev_random's "normal" is a bounded uniform."""
    host = oracle.fill_normal(dtype, count, seed, stream, 0.0, sigma, nthreads=THREADS)
    return host, torch.from_numpy(host.view(np.int16)).cuda()


def test_config3_true_normal_inputs_full_size(hip, oracle):
    """Configuration 3 on the inputs it names: 8 x bf16 N(0, 1) from seed 2, 64 Mi elements (128 MiB) each -> 1
    output, and the f16 form with two outputs on a quarter of that."""
    import torch
    for dtype, n_out, count in (("bf16", 1, 1 << 26), ("f16", 2, 1 << 24)):
        pairs = [_normal_on_device(torch, oracle, dtype, count, 2, k, 1.0) for k in range(8)]
        h_ins, d_ins = [p[0] for p in pairs], [p[1] for p in pairs]
        assert max(float(np.abs(oracle.widen(dtype, a[:1 << 22])).max()) for a in h_ins) > 4.5, "no tails: not a normal sample"
        outs = [torch.zeros(count, dtype=torch.int16, device="cuda") for _ in range(n_out)]
        hip.reduce_copy(dtype, "sum", d_ins, outs, count, _stream(torch))
        torch.cuda.synchronize()
        want = _expect(oracle, dtype, "sum", h_ins)
        for j, o in enumerate(outs):
            H.assert_bits_equal(o.cpu().numpy().view(np.uint16), want, "%s 8->%d output %d on N(0,1) inputs" % (dtype, n_out, j))
        del pairs, h_ins, d_ins, outs


def test_config2_true_normal_inputs_full_size(hip, oracle):
    """Configuration 2 on the inputs it names: bf16 N(0, 1e-2) from seed 1, one rank's 14 ring steps over
    32 MiB chunks, as 14 launches and as one launch of the queue executor; both against the CPU checker."""
    import torch
    W, ce = 8, 1 << 24
    h_grad, grad = _normal_on_device(torch, oracle, "bf16", W * ce, 1, 0, 1e-2)
    peers = [_normal_on_device(torch, oracle, "bf16", ce, 1, 1 + s, 1e-2) for s in range(W - 1)]
    h_peers, d_peers = [p[0] for p in peers], [p[1] for p in peers]
    h_result = np.zeros(W * ce, dtype=np.uint16)
    h_send = None
    for s in range(W - 1):
        c = (W - 1 - s) % W
        h_send = _expect(oracle, "bf16", "sum", [h_peers[s], h_grad[c * ce:(c + 1) * ce]])
        h_result[c * ce:(c + 1) * ce] = h_send
    for s in range(W - 1):
        c = (W - s) % W
        h_result[c * ce:(c + 1) * ce] = h_peers[s]
    result = torch.zeros(W * ce, dtype=torch.int16, device="cuda")
    send = torch.zeros(ce, dtype=torch.int16, device="cuda")
    ops = []
    for s in range(W - 1):
        c = (W - 1 - s) % W
        ops.append(dict(dtype="bf16", compute="sum", ins=[d_peers[s], grad[c * ce:(c + 1) * ce]],
                        outs=[result[c * ce:(c + 1) * ce], send], count=ce, deps=[len(ops) - 1] if ops else []))
    for s in range(W - 1):
        c = (W - s) % W
        ops.append(dict(dtype="bf16", compute="sum", ins=[d_peers[s]], outs=[result[c * ce:(c + 1) * ce]], count=ce,
                        deps=[s - 1] if s else []))
    for o in ops:
        hip.reduce_copy("bf16", "sum", o["ins"], o["outs"], ce, _stream(torch))
    torch.cuda.synchronize()
    H.assert_bits_equal(result.cpu().numpy().view(np.uint16), h_result, "14 launches, assembled 256 MiB result")
    H.assert_bits_equal(send.cpu().numpy().view(np.uint16), h_send, "14 launches, send buffer")
    result.zero_()
    send.zero_()
    g = hip.Graph(ops)
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (14, 14)
    H.assert_bits_equal(result.cpu().numpy().view(np.uint16), h_result, "one queue launch, assembled 256 MiB result")
    H.assert_bits_equal(send.cpu().numpy().view(np.uint16), h_send, "one queue launch, send buffer")
    g.destroy()


# forced members of the count list plus a log-uniform draw from [1, 2^28] (seed 3)
FORCED = [1, 2, 3, 5, 7, 31, 127, 8191, 131071, 524287, (1 << 20) + 7, (1 << 24) - 3, (1 << 28) - 57, 1 << 28]


def _config4_counts(oracle):
    extra = []
    for i in range(6):
        u = (oracle.rng_u64(3, 99, i) >> 11) / float(1 << 53)
        extra.append(max(1, int(2.0 ** (28.0 * u))))
    return FORCED + extra


@pytest.mark.parametrize("dtype, compute", [("i32", "sum"), ("i32", "max"), ("f32", "min"), ("f32", "prod")])
def test_config4_unaligned_mixed_ops(hip, oracle, dtype, compute):
    """4 inputs -> 1 output; every buffer sits 4..60 bytes past a 64-byte boundary, independently;
    counts include 1, primes and 2^28."""
    import torch
    counts = _config4_counts(oracle)
    big = max(counts)
    kind = "uniform" if dtype == "f32" else "normal"
    pool = [_dev_random(torch, dtype, big + 64, 3000 + k, kind=kind) for k in range(4)]
    out_pool = torch.zeros((big + 64) * 4 + 256, dtype=torch.uint8, device="cuda")
    h_pool = [_host(p, dtype) for p in pool]
    assert all(p.data_ptr() % 64 == 0 for p in pool) and out_pool.data_ptr() % 64 == 0
    for ci, count in enumerate(counts):
        offs = [4 * (1 + (oracle.rng_u64(3, 7, ci * 8 + k) % 15)) for k in range(5)]  # 4..60 bytes
        assert all(4 <= o <= 60 for o in offs)
        in_ptrs = [pool[k].data_ptr() + offs[k] for k in range(4)]
        out_ptr = out_pool.data_ptr() + 64 + offs[4]
        guard_lo = out_pool[:64 + offs[4]].clone()
        hip.reduce_copy(dtype, compute, in_ptrs, [out_ptr], count, _stream(torch))
        torch.cuda.synchronize()
        h_ins = [h_pool[k][offs[k] // 4: offs[k] // 4 + count] for k in range(4)]
        want = _expect(oracle, dtype, compute, [np.ascontiguousarray(a) for a in h_ins])
        lo = 64 + offs[4]
        got = out_pool[lo:lo + 4 * count].cpu().numpy().view(NPDT[dtype])
        H.assert_bits_equal(got, want, "%s %s count=%d offsets=%s" % (dtype, compute, count, offs))
        assert torch.equal(out_pool[:lo], guard_lo), "bytes before the output were touched"
        assert int(out_pool[lo + 4 * count: lo + 4 * count + 64].max()) == 0, "bytes after the output were touched"
        out_pool[lo:lo + 4 * count].zero_()


def test_config5_small_message_schedule_full_size(hip, oracle):
    """4096 ops (36 ring all-reduces over 8 virtual ranks + 64 copies), bf16 sum, op sizes log-uniform in
    [8 KiB, 256 KiB], one persistent launch; compared with the checker replaying the op list."""
    import torch
    import schedules as S
    from pccl_amd import lang
    ir, per = lang.small_message_allreduce()
    low = ir.lower()
    assert len(low) == 4096
    sizes_b = [o["count"] * 2 for o in low]
    assert min(sizes_b) >= 8 << 10 and max(sizes_b) <= 256 << 10
    d_in = [_dev_random(torch, "bf16", per, 4000 + r) for r in range(8)]
    d_out = [torch.zeros(per, dtype=torch.bfloat16, device="cuda") for _ in range(8)]
    dev = {"in": d_in, "out": d_out}
    g = hip.Graph(lang.bind(low, lambda b, r, e: dev[b][r].data_ptr() + 2 * e))
    h = {"in": [_host(t, "bf16") for t in d_in], "out": [np.zeros(per, dtype=np.uint16) for _ in range(8)]}
    order = oracle.topo_sort(len(low), [(d, i) for i, o in enumerate(low) for d in o["deps"]])
    host_ops = [dict(o, ins=[h[b][r][e:e + o["count"]] for (b, r, e) in o["ins"]],
                     outs=[h[b][r][e:e + o["count"]] for (b, r, e) in o["outs"]]) for o in low]
    oracle.run_ops(host_ops, order)
    for it in range(3):
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (4096, 4096)
        for r in range(8):
            H.assert_bits_equal(_host(d_out[r], "bf16"), h["out"][r], "run %d rank %d" % (it, r))
        for t in d_out:
            t.zero_()
    g.destroy()


def test_buffers_beyond_4_gib(hip):
    """Single operands larger than 4 GiB: every byte offset inside the kernels must be 64-bit.
    Checked on the device against torch (i32 sums wrap the same way; a copy is byte equality),
    at both ends and around the 4 GiB mark, for the direct launch and the queue executor."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    n = (1 << 30) + 4099                      # int32 elements: 4 GiB + 16 KiB + 12 B
    a = torch.randint(-(1 << 31), (1 << 31) - 1, (n + 1,), dtype=torch.int32, device="cuda")
    b = torch.randint(-(1 << 31), (1 << 31) - 1, (n + 1,), dtype=torch.int32, device="cuda")
    out = torch.zeros(n + 2, dtype=torch.int32, device="cuda")
    windows = [slice(0, 1 << 20), slice((1 << 30) - (1 << 19), (1 << 30) + 4099)]

    def check(got, want, what):
        for w in windows:
            assert torch.equal(got[w], want[w]), what
        # and a strided sample across the whole range
        assert torch.equal(got[::4099], want[::4099]), what

    # aligned operands
    hip.reduce_copy("i32", "sum", [a[:n], b[:n]], [out[:n]], n, stream)
    torch.cuda.synchronize()
    check(out[:n], a[:n] + b[:n], "aligned 2 -> 1 beyond 4 GiB")
    # unaligned operands (4 bytes off) and a copy
    out.zero_()
    hip.reduce_copy("i32", "sum", [a[1:]], [out[2:]], n, stream)
    torch.cuda.synchronize()
    check(out[2:], a[1:], "unaligned copy beyond 4 GiB")
    assert int(out[0]) == 0 and int(out[1]) == 0
    # the queue executor on the same operands
    out.zero_()
    g = hip.Graph([dict(dtype="i32", compute="sum", ins=[a[1:], b[:n]], outs=[out[:n]], count=n)])
    g.run(stream)
    assert g.status(stream) == (1, 1)
    check(out[:n], a[1:] + b[:n], "queue 2 -> 1 beyond 4 GiB")
    assert int(out[n]) == 0
    g.destroy()
    del a, b, out
    torch.cuda.empty_cache()


@pytest.mark.parametrize("dtype", ["bf16", "f16"])
def test_two_byte_offsets_at_16_mi_elements(hip, oracle, dtype):
    """The unaligned stress of configuration 4 for the 2-byte types: four inputs and the output each start an
    odd number of elements (2, 6, 10 ... bytes) off a 64-byte line, 2^24 + 7 elements, sum and max."""
    import torch
    count = (1 << 24) + 7
    offs = [2, 6, 14, 30, 62]          # bytes; the output's (last) differs from every input's
    pool = [_dev_random(torch, dtype, count + 64, 40 + k, kind="uniform", lo=-2.0, hi=2.0) for k in range(4)]
    out = torch.zeros(count + 64, dtype=pool[0].dtype, device="cuda")
    ptr_in = [pool[k].data_ptr() + offs[k] for k in range(4)]
    host_ins = [_host(pool[k], dtype)[offs[k] // 2:offs[k] // 2 + count] for k in range(4)]
    for compute in ("sum", "max"):
        out.zero_()
        hip.reduce_copy(dtype, compute, ptr_in, [out.data_ptr() + offs[4]], count, _stream(torch))
        torch.cuda.synchronize()
        got = _host(out, dtype)
        H.assert_bits_equal(got[offs[4] // 2:offs[4] // 2 + count], _expect(oracle, dtype, compute, host_ins),
                            "%s %s at 2-byte offsets" % (dtype, compute))
        assert not got[:offs[4] // 2].any() and not got[offs[4] // 2 + count:].any(), "wrote outside the output"
