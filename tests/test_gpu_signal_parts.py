"""Signals of a word per part (pccl_op_desc::signal_parts): a NOTIFY / GET_NOTIFIED pair whose signal is K
words, word p standing for part p of the data.  The data op that carries such a signal is cut into K parts;
whoever completes part p stores word p, and part p of the consumer polls word p only, so a ring whose ranks
are linked by signal words alone streams part by part.  Bit for bit what the CPU checker gives for the same
ops in program order."""
import numpy as np
import pytest

import helpers as H
from test_gpu_capture import _capture

pytestmark = pytest.mark.gpu


def _stream(torch):
    return torch.cuda.current_stream().cuda_stream


def _signalled_ring(torch, hip, oracle, world, size, parts, seed, first_slot=0):
    """(graph, bound ops, device buffers, expected per-rank outputs, signal words) of a ring all-reduce linked by
    signals of `parts` words."""
    from pccl_amd import lang
    ir, per_rank = lang.ring_allreduce_signalled(world, size, dtype="bf16", first_slot=first_slot, signal_parts=parts)
    low = ir.lower()
    words = torch.zeros(256, dtype=torch.int32, device="cuda")
    bufs = {"in": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(world)],
            "out": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(world)]}
    bound = lang.bind(low, lambda b, r, e: bufs[b][r].ptr + 2 * e, signals=words.data_ptr())

    def expect(host_in):
        outs = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
        hb = {"in": host_in, "out": outs}
        for o in low:            # creation order is each rank's program order, steps ascending: a valid order
            if o["primitive"] >= 2:
                continue
            n = o["count"]
            oracle.reduce_copy("bf16", "sum", [hb[b][r][e:e + n] for (b, r, e) in o["ins"]], [hb[b][r][e:e + n] for (b, r, e) in o["outs"]])
        return outs

    return low, bound, bufs, expect, words, per_rank


@pytest.mark.parametrize("world,size,parts", [(8, 20_011, 8), (8, 100, 8), (4, 300_007, 32), (8, 3_001, 2), (3, 65_536, 16)])
def test_ring_linked_by_signals_of_a_word_per_part(hip, oracle, world, size, parts):
    """(size 100 with 8 parts: parts 2..7 of every op are empty and still have to pass their word on.)"""
    import torch
    low, bound, bufs, expect, words, per_rank = _signalled_ring(torch, hip, oracle, world, size, parts, 0)
    carrier, cut = hip.plan_signals(bound, with_parts=True)
    n_signal = sum(1 for o in low if o["primitive"] >= 2)
    assert sum(1 for c in carrier if c >= 0) == n_signal and set(cut) == {parts}     # every signal op rides, every data op is cut into `parts`
    g = hip.Graph(bound)
    assert g.info()["n_tiles"] == parts * (len(low) - n_signal)
    for it in range(2):
        host_in = [H.gen("bf16", per_rank, 700 + it, r) for r in range(world)]
        want = expect(host_in)
        for r in range(world):
            bufs["in"][r].upload(host_in[r])
            bufs["out"][r].view().fill_(0xFF)
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (len(low), len(low))
        for r in range(world):
            H.assert_bits_equal(bufs["out"][r].download(), want[r], "world %d size %d parts %d, run %d rank %d" % (world, size, parts, it, r))
            assert bufs["out"][r].guards_intact()
        # every word of every link holds the last step's value of this run
        base = (it + 1) << 16
        got = words[:world * parts].cpu().tolist()
        assert got == [base + 2 * world - 2] * (world * parts)
    g.destroy()


def test_replay_and_rebind_of_a_ring_linked_by_per_part_signals(hip, oracle):
    """Recorded once by stream capture and replayed on fresh inputs (every replay takes a fresh run number from
    the device); then the output buffers move (graph_rebind) and the same recording is replayed again."""
    import torch
    world, size, parts = 8, 5_003, 4
    low, bound, bufs, expect, words, per_rank = _signalled_ring(torch, hip, oracle, world, size, parts, 0, first_slot=32)
    g = hip.Graph(bound)
    graph = _capture(torch, lambda stream: g.run(stream))
    stream = _stream(torch)
    for it in range(3):
        host_in = [H.gen("bf16", per_rank, 720 + it, r) for r in range(world)]
        want = expect(host_in)
        for r in range(world):
            bufs["in"][r].upload(host_in[r])
            bufs["out"][r].view().fill_(0xFF)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert g.status(stream) == (len(low), len(low))
        for r in range(world):
            H.assert_bits_equal(bufs["out"][r].download(), want[r], "replay %d rank %d" % (it, r))
    # new output buffers for ranks 0 and 5, and the signal words move too
    moved = {r: H.DevBuf(torch, "bf16", per_rank, 0) for r in (0, 5)}
    for r, nb in moved.items():
        g.rebind(bufs["out"][r].ptr, nb.ptr, 2 * per_rank, stream)
    words2 = torch.zeros(256, dtype=torch.int32, device="cuda")
    g.rebind(words.data_ptr(), words2.data_ptr(), 4 * 256, stream)
    outs = [moved.get(r, bufs["out"][r]) for r in range(world)]
    for it in range(2):
        host_in = [H.gen("bf16", per_rank, 740 + it, r) for r in range(world)]
        want = expect(host_in)
        for r in range(world):
            bufs["in"][r].upload(host_in[r])
            outs[r].view().fill_(0xFF)
        words.zero_()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert g.status(stream) == (len(low), len(low))
        for r in range(world):
            H.assert_bits_equal(outs[r].download(), want[r], "after the rebind, replay %d rank %d" % (it, r))
            assert outs[r].guards_intact()
        assert int(words.abs().sum()) == 0 and int((words2[32:32 + world * parts] != 0).sum()) == world * parts
    g.destroy()


def test_per_part_signals_that_no_data_op_carries(hip, oracle):
    """t = a + b and u = a * ... two ops in front of ONE NOTIFY of 8 words, and two ops behind ONE GET_NOTIFIED of 8
    words: neither signal op can ride on a data op, so the NOTIFY stores all 8 words once both ops are complete
    and the GET_NOTIFIED waits for all 8.  And an op between a wait of 8 words and a notify of 4: it carries the
    notify (4 parts), the wait stays an op of its own."""
    import torch
    n = 40_003
    a, b = H.gen("f32", n, 760, 0), H.gen("f32", n, 760, 1)
    da, db = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0, src=b)
    dt, du, dv, dw, dx = (H.DevBuf(torch, "f32", n, 0) for _ in range(5))
    sig = torch.zeros(64, dtype=torch.int32, device="cuda")
    s0, s1 = sig.data_ptr(), sig.data_ptr() + 4 * 16
    ops = [dict(dtype="f32", compute="sum", ins=[da.ptr, db.ptr], outs=[dt.ptr], count=n, deps=[]),            # 0
           dict(dtype="f32", compute="max", ins=[da.ptr, db.ptr], outs=[du.ptr], count=n, deps=[]),            # 1
           dict(primitive=hip.NOTIFY, signal=s0, value=3, parts=8, deps=[0, 1]),                               # 2: behind two ops
           dict(primitive=hip.GET_NOTIFIED, signal=s0, value=3, parts=8, deps=[]),                             # 3: two ops wait for it
           dict(dtype="f32", compute="sum", ins=[dt.ptr, du.ptr], outs=[dv.ptr], count=n, deps=[3]),           # 4
           dict(dtype="f32", compute="min", ins=[dt.ptr, du.ptr], outs=[dw.ptr], count=n, deps=[3]),           # 5
           dict(primitive=hip.NOTIFY, signal=s1, value=1, parts=4, deps=[4]),                                  # 6: rides on op 4
           dict(primitive=hip.GET_NOTIFIED, signal=s1, value=1, parts=4, deps=[]),                             # 7: rides on op 8
           dict(dtype="f32", compute="sum", ins=[dv.ptr], outs=[dx.ptr], count=n, deps=[7])]                   # 8
    carrier, cut = hip.plan_signals(ops, with_parts=True)
    assert carrier == [-1, -1, -1, -1, -1, -1, 4, 8, -1] and cut == [0, 0, 0, 0, 4, 0, 4, 4, 4]
    g = hip.Graph(ops)
    t, u = oracle.reduce("f32", "sum", [a, b]), oracle.reduce("f32", "max", [a, b])
    v, w = oracle.reduce("f32", "sum", [t, u]), oracle.reduce("f32", "min", [t, u])
    for run in range(2):
        for d in (dt, du, dv, dw, dx):
            d.view().fill_(0xFF)
        g.run(_stream(torch))
        assert g.status(_stream(torch)) == (9, 9)
        for d, want, name in ((dt, t, "t"), (du, u, "u"), (dv, v, "v"), (dw, w, "w"), (dx, v, "x")):
            H.assert_bits_equal(d.download(), want, "run %d: %s" % (run, name))
            assert d.guards_intact()
        base = (run + 1) << 16
        got = sig.cpu().tolist()
        assert got[:8] == [base + 3] * 8 and got[16:20] == [base + 1] * 4 and not any(got[8:16]) and not any(got[20:])
    g.destroy()


def test_a_part_whose_word_never_comes_gives_up_and_the_graph_recovers(hip, oracle):
    """The host plays the producer of a GET_NOTIFIED of 4 words and leaves word 2 out: part 2 of the copy behind it
    gives up (spin limit set from the host, every workgroup leaves normally), status reports PCCL_ERR_GRAPH and
    restores the graph; with all four words stored the next run is complete and correct."""
    import torch
    n = 100_000
    src = H.gen("f32", n, 770, 0)
    x, y = H.DevBuf(torch, "f32", n, 0, src=src), H.DevBuf(torch, "f32", n, 0)
    sig = torch.zeros(8, dtype=torch.int32, device="cuda")
    ops = [dict(primitive=hip.GET_NOTIFIED, signal=sig.data_ptr(), value=5, parts=4, deps=[]),
           dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=n, deps=[0])]
    g = hip.Graph(ops)
    g.set_spin_limit(20000)
    base = g.next_signal_base()
    sig[:4] = torch.tensor([base + 5, base + 5, 0, base + 5], dtype=torch.int64).to(torch.int32)
    torch.cuda.synchronize()
    g.run(_stream(torch))
    with pytest.raises(hip.PcclError) as e:
        g.status(_stream(torch))
    assert e.value.code == hip.ERR_GRAPH
    per = hip.part_elems(n, 4)
    got = y.download()
    H.assert_bits_equal(got[:2 * per], src[:2 * per], "parts 0 and 1 ran")
    H.assert_bits_equal(got[3 * per:], src[3 * per:], "part 3 ran")
    assert bool((y.view()[4 * 2 * per:4 * 3 * per] == 0xFF).all()), "part 2 must not have run: its word never came"
    base = g.next_signal_base()
    sig[:4] = base + 5
    y.view().fill_(0xFF)
    torch.cuda.synchronize()
    g.run(_stream(torch))
    assert g.status(_stream(torch)) == (2, 2)
    H.assert_bits_equal(y.download(), src, "after the reset")
    g.destroy()
