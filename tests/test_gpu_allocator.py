"""The plugin's allocator on the GPU: 2 MiB-rounded allocations tracked by pointer (the role of
csrc/plugins/cuda_executor/device.cc:59-144)."""
import numpy as np
import pytest

import helpers as H

pytestmark = pytest.mark.gpu

MIB = 1 << 20


def _fill_and_check(torch, hip, ptrs, nbytes):
    """Every buffer gets its own byte pattern; all are read back afterwards (nothing overlaps)."""
    stream = torch.cuda.current_stream().cuda_stream
    srcs = []
    for k, p in enumerate(ptrs):
        src = torch.full((nbytes,), (17 * k + 3) & 0xFF, dtype=torch.uint8, device="cuda")
        hip.reduce_copy("f8e4m3", "sum", [src], [p], nbytes, stream)
        srcs.append(src)
    back = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    for k, p in enumerate(ptrs):
        hip.reduce_copy("f8e4m3", "sum", [p], [back], nbytes, stream)
        torch.cuda.synchronize()
        assert torch.equal(back, srcs[k]), "buffer %d was overwritten" % k


def test_allocations_are_disjoint_aligned_and_tracked(hip):
    import torch
    sizes = [100, 3 * MIB + 5, 16 * MIB, 40 * MIB, 16 * MIB, 2 * MIB]
    ptrs = [hip.alloc(n) for n in sizes]
    assert all(p % 4096 == 0 for p in ptrs)
    # every allocation has its size rounded up to 2 MiB to itself
    spans = sorted((p, p + (n + 2 * MIB - 1) // (2 * MIB) * (2 * MIB)) for p, n in zip(ptrs, sizes))
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))
    _fill_and_check(torch, hip, ptrs, 100)
    # the last bytes of a rounded allocation are usable
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.arange(256, dtype=torch.uint8, device="cuda")
    end = ptrs[1] + 4 * MIB - 256
    hip.reduce_copy("f8e4m3", "sum", [src], [end], 256, stream)
    back = torch.empty_like(src)
    hip.reduce_copy("f8e4m3", "sum", [end], [back], 256, stream)
    torch.cuda.synchronize()
    assert torch.equal(back, src)
    hip.free(ptrs[2])
    hip.free(ptrs[3])
    again = hip.alloc(50 * MIB)
    _fill_and_check(torch, hip, [ptrs[0], ptrs[1], ptrs[4], ptrs[5], again], 100)
    for p in (ptrs[0], ptrs[1], ptrs[4], ptrs[5], again):
        hip.free(p)
    with pytest.raises(hip.PcclError):
        hip.free(ptrs[0])          # already gone
    with pytest.raises(hip.PcclError):
        hip.free(again + 4096)     # not the start of an allocation
    with pytest.raises(hip.PcclError):
        hip.alloc(0)
    hip.free(0)                    # (a null pointer is fine, as for hipFree)


def test_large_buffers_allocated_one_by_one_hold_operands(hip, oracle):
    """Nine 64 MiB buffers from nine calls hold data independently and a fold over them is bit-exact."""
    import torch
    n, count = 9, 32 * MIB          # bf16 elements: 64 MiB per buffer
    ptrs = [hip.alloc(2 * count) for _ in range(n)]
    assert all(p % 4096 == 0 for p in ptrs) and all(abs(a - b) >= 2 * count for a in ptrs for b in ptrs if a != b)
    stream = torch.cuda.current_stream().cuda_stream
    ins = [H.gen("bf16", count, 77, k) for k in range(n - 1)]
    for a, p in zip(ins, ptrs):
        t = torch.from_numpy(a.view(np.int16)).cuda()
        hip.reduce_copy("bf16", "sum", [t], [p], count, stream)
    hip.reduce_copy("bf16", "sum", ptrs[:n - 1], [ptrs[n - 1]], count, stream)
    got = torch.empty(count, dtype=torch.int16, device="cuda")
    hip.reduce_copy("bf16", "sum", [ptrs[n - 1]], [got], count, stream)
    torch.cuda.synchronize()
    H.assert_bits_equal(got.cpu().numpy().view(np.uint16), oracle.reduce("bf16", "sum", ins), "fold over plugin-allocated buffers")
    for p in ptrs:
        hip.free(p)
