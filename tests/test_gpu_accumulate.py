"""GPU parity of pccl_hip_accumulate (fold one input into K destinations) against the CPU checker
applying the same two-input fold, destination first, to every destination."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", ["f32", "i32", "bf16", "f16", "f64", "u32"])
@pytest.mark.parametrize("compute", ["sum", "prod", "min", "max"])
def test_accumulate_matches_checker(hip, oracle, dtype, compute):
    import torch
    es = H.ELEM_BYTES[dtype]
    for count, n_out, offs in ((1, 1, [0, 0]), (7, 2, [0, 0, 0]), (100003, 3, [0, 0, 0, 0]),
                               (70001, 2, [es, 3 * es, 5 * es]), (1 << 20, 8, [0] * 9), (4099, 8, [es * k for k in range(9)])):
        kind = dict(kind="uniform", lo=0.5, hi=2.0) if compute == "prod" and dtype not in ("i32", "u32") else {}
        kw = dict(lo=-7, hi=7) if compute == "prod" and dtype == "i32" else kind
        kw = dict(lo=0, hi=13) if compute == "prod" and dtype == "u32" else kw
        src = H.gen(dtype, count, 200, 0, **kw)
        dsts = [H.gen(dtype, count, 200, 1 + j, **kw) for j in range(n_out)]
        want = [oracle.reduce(dtype, compute, [d, src]) for d in dsts]
        d_src = H.DevBuf(torch, dtype, count, offs[0], src=src)
        d_dst = [H.DevBuf(torch, dtype, count, offs[1 + j], src=dsts[j]) for j in range(n_out)]
        hip.accumulate(dtype, compute, d_src.ptr, [b.ptr for b in d_dst], count, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for j in range(n_out):
            H.assert_bits_equal(d_dst[j].download(), want[j], "%s %s count=%d dst %d/%d" % (dtype, compute, count, j, n_out))
            assert d_dst[j].guards_intact()
        H.assert_bits_equal(d_src.download(), src, "input untouched")


def test_accumulate_order_is_destination_first(hip, oracle):
    """min/max keep the accumulator on ties and NaN rules depend on operand order: destination is
    the accumulator.  (1e8 + 1) style case for sum: dst=1e8, value=1 -> 1e8."""
    import torch
    dst = np.array([1e8, 1.0, -0.0, 0.0], dtype=np.float32)
    src = np.array([1.0, 1e8, 0.0, -0.0], dtype=np.float32)
    for compute in ("sum", "min", "max"):
        want = oracle.reduce("f32", compute, [dst, src])
        d_s, d_d = H.DevBuf(torch, "f32", 4, 0, src=src), H.DevBuf(torch, "f32", 4, 0, src=dst)
        hip.accumulate("f32", compute, d_s.ptr, [d_d.ptr], 4)
        torch.cuda.synchronize()
        H.assert_bits_equal(d_d.download(), want, compute)


def test_accumulate_errors(hip):
    import torch
    t = torch.zeros(64, dtype=torch.float32, device="cuda")
    u = torch.zeros(64, dtype=torch.float32, device="cuda")
    with pytest.raises(hip.PcclError) as e:
        hip.accumulate("f32", "sum", t, [u, u], 8)
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.accumulate("f32", "sum", t, [], 8)
    assert e.value.code == hip.ERR_INVALID_ARG
    with pytest.raises(hip.PcclError) as e:
        hip.accumulate("f32", "sum", t.data_ptr() + 2, [u], 8)
    assert e.value.code == hip.ERR_MISALIGNED
    with pytest.raises(hip.PcclError) as e:
        hip.accumulate(99, "sum", t, [u], 8)
    assert e.value.code == hip.ERR_UNSUPPORTED
    hip.accumulate("f32", "sum", t, [u], 0)


def test_cache_treatments_through_the_knob(hip, oracle):
    """Cache treatment 0 / 1 / 2 (chosen from operand sizes in normal use) forced on small inputs."""
    import torch
    n = 70001
    try:
        for dtype, n_out, off in (("bf16", 1, 0), ("bf16", 3, 2), ("f32", 2, 4), ("f8e5m2", 7, 1)):
            src = H.gen(dtype, n, 70, 0)
            dst0 = [H.gen(dtype, n, 70, 1 + k) for k in range(n_out)]
            for mem in (0, 1, 2):
                hip.set_tuning(0, mem)
                d_src = H.DevBuf(torch, dtype, n, src=src, offset=off)
                d_dst = [H.DevBuf(torch, dtype, n, src=x, offset=(off * (k + 1)) % 64) for k, x in enumerate(dst0)]
                hip.accumulate(dtype, "sum", d_src.ptr, [x.ptr for x in d_dst], n, torch.cuda.current_stream().cuda_stream)
                torch.cuda.synchronize()
                for k, x in enumerate(d_dst):
                    H.assert_bits_equal(x.download(), oracle.reduce(dtype, "sum", [dst0[k], src]),
                                        "%s 1->%d mem=%d dst %d" % (dtype, n_out, mem, k))
                    assert x.guards_intact()
    finally:
        hip.set_tuning(0, -1)
