"""The asynchronous entry points recorded into a HIP graph by stream capture (torch.cuda.graph)
and replayed: they allocate nothing, synchronise nothing and enqueue no memset, so a replay is
just their kernels.  Every replay runs on fresh inputs, with eager work and synchronisation in
between, and is checked bit for bit against the CPU checker."""
import numpy as np
import pytest

import helpers as H
from test_gpu_graph import _signal_ring_ops

pytestmark = pytest.mark.gpu


def _capture(torch, record):
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        record(side.cuda_stream)            # warm-up on the capture stream (module load etc.)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        record(torch.cuda.current_stream().cuda_stream)
    return graph


def test_reduce_copy_and_accumulate_replay(hip, oracle):
    import torch
    n = 1_000_003
    d_in = [H.DevBuf(torch, "bf16", n, offset=2 * k) for k in range(3)]
    d_sum = H.DevBuf(torch, "bf16", n)
    d_acc = [H.DevBuf(torch, "bf16", n, offset=4), H.DevBuf(torch, "bf16", n)]

    def record(stream):
        hip.reduce_copy("bf16", "sum", [b.ptr for b in d_in], [d_sum.ptr], n, stream)
        hip.accumulate("bf16", "sum", d_sum.ptr, [b.ptr for b in d_acc], n, stream)

    graph = _capture(torch, record)
    for it in range(3):
        ins = [H.gen("bf16", n, 200 + it, k) for k in range(3)]
        acc0 = [H.gen("bf16", n, 200 + it, 3 + k) for k in range(2)]
        for b, a in zip(d_in + d_acc, ins + acc0):
            b.upload(a)
        d_sum.view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = oracle.reduce("bf16", "sum", ins)
        H.assert_bits_equal(d_sum.download(), want, "replay %d sum" % it)
        for k in range(2):
            H.assert_bits_equal(d_acc[k].download(), oracle.reduce("bf16", "sum", [acc0[k], want]),
                                "replay %d destination %d" % (it, k))
            assert d_acc[k].guards_intact()


def test_queue_run_with_signal_ops_replay(hip, oracle):
    """A ring whose virtual ranks are linked only by NOTIFY / GET_NOTIFIED, recorded once: each
    replay must use a fresh run number, or the waits would be satisfied by the previous replay's
    signal values before the data is there."""
    import torch
    world, size = 8, 3001
    per = world * size
    d_in = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    d_out = [H.DevBuf(torch, "bf16", per, 0) for _ in range(world)]
    signals = torch.zeros(64, dtype=torch.int32, device="cuda")
    ops, sym = _signal_ring_ops(world, size, signals.data_ptr(), d_in, d_out)
    g = hip.Graph(ops)
    graph = _capture(torch, lambda stream: g.run(stream))   # the warm-up inside is run 1, the recording run 2
    seen = []
    for it in range(3):
        ins = [H.gen("bf16", per, 300 + 10 * it, r) for r in range(world)]
        outs = [np.zeros(per, dtype=np.uint16) for _ in range(world)]
        bufs = {"in": ins, "out": outs}
        for i in sorted(sym):
            o = sym[i]
            oracle.reduce_copy("bf16", "sum", [bufs[b][r][e:e + size] for (b, r, e) in o["ins"]],
                               [bufs[b][r][e:e + size] for (b, r, e) in o["outs"]])
        for r in range(world):
            d_in[r].upload(ins[r])
            d_out[r].view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert g.status(torch.cuda.current_stream().cuda_stream) == (len(ops), len(ops))
        for r in range(world):
            H.assert_bits_equal(d_out[r].download(), outs[r], "replay %d rank %d" % (it, r))
        word = signals[:world].cpu().tolist()
        assert len(set(word)) == 1
        seen.append(word[0])
    # consecutive replays used consecutive run numbers
    assert [b - a for a, b in zip(seen, seen[1:])] == [1 << 16, 1 << 16]
    g.destroy()


def test_recorded_queue_run_survives_a_rebind_that_changes_aliasing(hip, oracle, monkeypatch):
    """A: t = a + b; B: u = t + c, recorded once.  Rebinding u onto a's buffer (shifted) turns
    the dependency from part-by-part to whole-op, which rebuilds the graph's contents; the
    recording made before must still be valid (same arena) and give sequential results."""
    import torch
    monkeypatch.setenv("PCCL_HIP_WIDE", "0")  # (the persistent drain; a wide launch refuses such a rebind)
    count, shift = 1500 * 1000, 64
    a_full = H.gen("f32", count + shift, 401, 0)
    b, c = H.gen("f32", count, 401, 1), H.gen("f32", count, 401, 2)
    dA = H.DevBuf(torch, "f32", count + shift, 0, src=a_full)
    db, dc = H.DevBuf(torch, "f32", count, 0, src=b), H.DevBuf(torch, "f32", count, 0, src=c)
    dt, du = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    g = hip.Graph([dict(dtype="f32", compute="sum", ins=[dA.ptr, db.ptr], outs=[dt.ptr], count=count, deps=[]),
                   dict(dtype="f32", compute="sum", ins=[dt.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[0])])
    assert g.dependency_kinds() == [1]
    arena = g.info()["device_layout"]
    graph = _capture(torch, lambda stream: g.run(stream))
    t = oracle.reduce("f32", "sum", [a_full[:count], b])
    u = oracle.reduce("f32", "sum", [t, c])
    du.view().fill_(0xFF)
    graph.replay()
    torch.cuda.synchronize()
    H.assert_bits_equal(du.download(), u, "replay before the rebind")
    g.rebind(du.ptr, dA.ptr + 4 * shift, 4 * count, torch.cuda.current_stream().cuda_stream)
    assert g.dependency_kinds() == [0] and g.info()["device_layout"] == arena
    for it in range(2):
        dA.upload(a_full)
        dt.view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        H.assert_bits_equal(dt.download(), t, "t, replay %d after the rebind" % it)
        H.assert_bits_equal(dA.download()[shift:], u, "u inside a's buffer, replay %d" % it)
    assert g.status(torch.cuda.current_stream().cuda_stream) == (2, 2)
    g.destroy()


def test_run_number_survives_a_rebuilding_rebind_after_replays(hip, oracle):
    """op0: t = a + b; NOTIFY; GET_NOTIFIED; op3: u = t + c (ordered after op0 only through the
    signal word); op4: v = u + d.  Recorded once and replayed three times, so the device's run
    number is ahead of the count of graph_run calls.  Moving v onto t (shifted) makes the edge
    op3 -> op4 whole-op, which rebuilds the arena: the rebuilt arena must go on from the device's
    run number.  Were it set back, the signal value left by an earlier replay would satisfy the
    wait at once and op3 would read t before op0 has written it."""
    import torch
    count, shift = 1500 * 1000, 64
    a, b, c, d = (H.gen("f32", count, 411, k) for k in range(4))
    da, db, dc, dd = (H.DevBuf(torch, "f32", count, 0, src=x) for x in (a, b, c, d))
    dT = H.DevBuf(torch, "f32", count + shift, 0)
    du, dv = H.DevBuf(torch, "f32", count, 0), H.DevBuf(torch, "f32", count, 0)
    sig = torch.zeros(4, dtype=torch.int32, device="cuda")
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dT.ptr], count=count, deps=[]),
           dict(primitive=2, signal=sig.data_ptr(), value=1, deps=[0]),
           dict(primitive=3, signal=sig.data_ptr(), value=1, deps=[]),
           dict(dtype="f32", compute="sum", ins=[dT.ptr, dc.ptr], outs=[du.ptr], count=count, deps=[2]),
           dict(dtype="f32", compute="sum", ins=[du.ptr, dd.ptr], outs=[dv.ptr], count=count, deps=[3])]
    g = hip.Graph(ops)
    assert g.dependency_kinds() == [0, 0, 1]
    graph = _capture(torch, lambda stream: g.run(stream))
    stream = torch.cuda.current_stream().cuda_stream
    t = oracle.reduce("f32", "sum", [a, b])
    u = oracle.reduce("f32", "sum", [t, c])
    v = oracle.reduce("f32", "sum", [u, d])
    words = []
    for it in range(3):
        for buf in (dT, du, dv):
            buf.view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        H.assert_bits_equal(dv.download(), v, "replay %d before the rebind" % it)
        words.append(int(sig[0].item()) & 0xffffffff)
    assert [y - x for x, y in zip(words, words[1:])] == [1 << 16, 1 << 16]
    g.rebind(dv.ptr, dT.ptr + 4 * shift, 4 * count, stream)   # v now overwrites what op3 reads, shifted
    assert g.dependency_kinds() == [0, 0, 0]
    # the host's idea of the next base follows the device from here (it counts graph_run calls, not replays)
    assert g.next_signal_base() == words[-1] - 1 + (1 << 16)
    for it in range(2):
        dT.view().fill_(0xFF)
        du.view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert g.status(stream) == (5, 5)
        H.assert_bits_equal(du.download(), u, "u, replay %d after the rebind" % it)
        H.assert_bits_equal(dT.download()[shift:], v, "v inside t's buffer, replay %d after the rebind" % it)
        words.append(int(sig[0].item()) & 0xffffffff)
    # the run number went on from where the device stood
    assert [y - x for x, y in zip(words, words[1:])] == [1 << 16] * 4
    g.destroy()
