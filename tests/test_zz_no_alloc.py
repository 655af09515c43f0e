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
