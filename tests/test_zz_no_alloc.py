"""pccl_hip_graph_run_static: the op-batching path with its device state in the library's fixed
per-GPU array instead of an allocated arena.  Checked against pccl_hip_graph_create / graph_run on the
same ops, bit for bit, and against the CPU checker; two calls in a row, the second smaller."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


def _ring_case(torch, hip, oracle, world, size, seed):
    """Ring all-reduce over `world` virtual ranks as a DAG (lang.ring_allreduce), operands bound to fresh buffers."""
    from pccl_amd import lang
    ir, per_rank = lang.ring_allreduce(world, size, dtype="bf16")
    low = ir.lower()
    host_in = [H.gen("bf16", per_rank, seed, r) for r in range(world)]

    def fresh():
        return {"in": [H.DevBuf(torch, "bf16", per_rank, 0, src=a) for a in host_in],
                "out": [H.DevBuf(torch, "bf16", per_rank, 0) for _ in range(world)]}

    def bind(bufs):
        return lang.bind(low, lambda b, r, e: bufs[b][r].ptr + 2 * e)

    # CPU checker: the ops in creation order (a valid order)
    outs = [np.zeros(per_rank, dtype=np.uint16) for _ in range(world)]
    hb = {"in": host_in, "out": outs}
    for o in low:
        n = o["count"]
        oracle.reduce_copy("bf16", "sum", [hb[b][r][e:e + n] for (b, r, e) in o["ins"]], [hb[b][r][e:e + n] for (b, r, e) in o["outs"]])
    return low, fresh, bind, outs


def _check_case(torch, hip, oracle, world, size, seed, what):
    stream = torch.cuda.current_stream().cuda_stream
    low, fresh, bind, want = _ring_case(torch, hip, oracle, world, size, seed)
    a, b = fresh(), fresh()
    g = hip.Graph(bind(a))                       # the existing entry points, allocated arena
    g.run(stream)
    assert g.status(stream) == (len(low), len(low))
    ops_b = bind(b)
    assert hip.graph_run_static(ops_b, stream) == (len(low), len(low))      # the fixed array
    for r in range(world):
        got_a, got_b = a["out"][r].download(), b["out"][r].download()
        H.assert_bits_equal(got_b, got_a, "%s: rank %d, static vs allocated arena" % (what, r))
        H.assert_bits_equal(got_b, want[r], "%s: rank %d vs CPU checker" % (what, r))
        assert b["out"][r].guards_intact()
    # the same ops again: no upload this time; the state in the array has re-armed itself
    for r in range(world):
        b["out"][r].view().fill_(0xFF)
    assert hip.graph_run_static(ops_b, stream, wait=False) is None
    torch.cuda.synchronize()
    for r in range(world):
        H.assert_bits_equal(b["out"][r].download(), want[r], "%s: rank %d, second run of the same ops" % (what, r))
    g.destroy()


def test_static_arena_matches_allocated_arena_twice_second_smaller(hip, oracle):
    import torch
    _check_case(torch, hip, oracle, 8, 40_003, 501, "first call")      # 112 ops of 80 KB
    _check_case(torch, hip, oracle, 4, 1_001, 502, "second, smaller call")   # 24 ops of 2 KB: state left by the first call must not matter


def test_static_arena_refuses_a_graph_beyond_its_size_and_works_afterwards(hip, oracle):
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    n = 1 << 24
    x = H.DevBuf(torch, "f32", n, 0, src=H.gen("f32", n, 503, 0))
    y = H.DevBuf(torch, "f32", n, 0, fill=0x5A)
    # four ops cut into 64 Ki parts of 1 KiB each: more queue entries than 8 MiB of state can hold
    ops = [dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=n, deps=[k - 1] if k else []) for k in range(4)]
    with pytest.raises(hip.PcclError) as e:
        hip.graph_run_static(ops, stream, tile_bytes=1024)
    assert "static arena" in str(e.value)
    torch.cuda.synchronize()
    assert bool((y.view() == 0x5A).all()), "a refused call must not launch anything"
    assert hip.graph_run_static([dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=n)], stream) == (1, 1)
    H.assert_bits_equal(y.download(), x.download(), "copy through the fixed array after a refused call")
    assert hip.graph_run_static([], stream) == (0, 0)


def test_a_run_that_gave_up_is_reported_by_the_next_call_and_the_one_after_runs_afresh(hip, oracle, monkeypatch):
    """A caller that passes no counters launches a graph whose GET_NOTIFIED nobody satisfies: the wait gives up
    inside the kernel (spin limit set from the host, every workgroup leaves normally).  The next call, same ops and
    again without counters, must not launch onto the abandoned state and return PCCL_OK with the outputs
    untouched: it reports PCCL_ERR_GRAPH.  The call after that, with the word satisfied, is a correct fresh run."""
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    monkeypatch.setenv("PCCL_HIP_SPIN_LIMIT_US", "20000")
    n = 50_000
    src = H.gen("f32", n, 504, 0)
    x = H.DevBuf(torch, "f32", n, 0, src=src)
    y = H.DevBuf(torch, "f32", n, 0, fill=0x5A)
    word = torch.zeros(4, dtype=torch.int32, device="cuda")
    ops = [dict(primitive=hip.GET_NOTIFIED, signal=word.data_ptr(), value=1, deps=[]),
           dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=n, deps=[0])]
    assert hip.graph_run_static(ops, stream, wait=False) is None      # gives up after 20 ms, unnoticed
    with pytest.raises(hip.PcclError) as e:
        hip.graph_run_static(ops, stream, wait=False)
    assert e.value.code == hip.ERR_GRAPH and "gave up" in str(e.value)
    torch.cuda.synchronize()
    assert bool((y.view() == 0x5A).all()), "nothing may have been copied: the signal never came"
    word.fill_(0x7fff0000)   # ahead of every run's signal base: the wait is satisfied at once
    torch.cuda.synchronize()
    assert hip.graph_run_static(ops, stream) == (2, 2)
    H.assert_bits_equal(y.download(), src, "fresh run after the abandoned one")
    assert y.guards_intact(0x5A)
    # ... and a caller that does pass counters hears of a wait that gave up in the same call
    word.zero_()
    torch.cuda.synchronize()
    with pytest.raises(hip.PcclError) as e:
        hip.graph_run_static(ops, stream)
    assert e.value.code == hip.ERR_GRAPH
    monkeypatch.delenv("PCCL_HIP_SPIN_LIMIT_US")
    assert hip.graph_run_static([dict(dtype="f32", compute="sum", ins=[x.ptr], outs=[y.ptr], count=n)], stream) == (1, 1)


def test_the_same_ops_on_another_stream_wait_for_the_run_before(hip, oracle):
    """Two calls with the same ops on two streams, nothing between them: the second waits for the first run
    (they share the one array) and both leave the checker's result."""
    import torch
    n = 1 << 22
    a, b = H.gen("f32", n, 505, 0), H.gen("f32", n, 505, 1)
    want = oracle.reduce("f32", "sum", [a, b])
    x, y = H.DevBuf(torch, "f32", n, 0, src=a), H.DevBuf(torch, "f32", n, 0, src=b)
    z = H.DevBuf(torch, "f32", n, 0, fill=0x5A)
    w = H.DevBuf(torch, "f32", n, 0, fill=0x5A)
    ops = [dict(dtype="f32", compute="sum", ins=[x.ptr, y.ptr], outs=[z.ptr], count=n, deps=[]),
           dict(dtype="f32", compute="sum", ins=[z.ptr], outs=[w.ptr], count=n, deps=[0])]
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    torch.cuda.synchronize()
    assert hip.graph_run_static(ops, s1.cuda_stream, wait=False) is None
    assert hip.graph_run_static(ops, s2.cuda_stream) == (2, 2)
    torch.cuda.synchronize()
    H.assert_bits_equal(z.download(), want, "fold")
    H.assert_bits_equal(w.download(), want, "copy behind it")
