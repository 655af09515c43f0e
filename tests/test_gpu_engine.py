"""GPU parity of the engine path: Engine.regOp(name, file) + Engine.exeOp(name, in, out) through
the host layer's C ABI, against the CPU checker replaying the same schedule file."""
import numpy as np
import pytest

import helpers as H
import schedules as S

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def E(hip):
    from pccl_amd import engine
    engine.lib()
    return engine


@pytest.fixture(scope="module")
def eng(E):
    e = E.Engine(0, 1)
    e.initEngine()
    yield e
    e.close()


def _oracle_replay(oracle, text, host_in):
    hdr, ops = S.parse_schedule_text(text)
    W, per = hdr["devices"], hdr["elems_per_device"]
    store = H.STORAGE[hdr["dtype"]]
    out = np.zeros(W * per, dtype=store)
    bufs = {"in": host_in, "out": out}
    order = oracle.topo_sort(len(ops), S.edges_of(ops))
    oracle.run_ops(S.materialise(ops, lambda b, r, e, n: bufs[b][r * per + e:r * per + e + n]), order)
    return hdr, out


def _to_dev(torch, a):
    return torch.from_numpy(a.view(np.uint8)).cuda()


def test_init_engine_workspace(eng):
    ws, sig, nbytes = eng.getDevBuffer("rocm")
    assert ws and nbytes == 1 << 28 and sig == ws + (1 << 28)   # 256 MiB + 256 int slots behind it
    assert ws % (2 << 20) == 0 or ws % 256 == 0


def test_ring_allreduce_from_native_file(E, eng, oracle, tmp_path):
    import torch
    p = str(tmp_path / "ring.sched")
    E.write_ring_allreduce(p, "bf16", "sum", 8, 12345)
    eng.regOp("ring", p)
    info = eng.opInfo("ring")
    n = info["devices"] * info["elems_per_device"]
    host_in = H.gen("bf16", n, 71, 0)
    hdr, want = _oracle_replay(oracle, open(p).read(), host_in)
    d_in, d_out = _to_dev(torch, host_in), torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    eng.exeOp("ring", d_in, d_out, stream)
    eng.waitOp("ring", stream)
    H.assert_bits_equal(d_out.cpu().numpy().view(np.uint16), want, "engine ring all-reduce")
    per = info["elems_per_device"]
    for r in range(1, 8):
        H.assert_bits_equal(want[r * per:(r + 1) * per], want[:per], "rank %d equals rank 0" % r)
    # new tensors: the graph is re-bound, not rebuilt
    host_in2 = H.gen("bf16", n, 72, 0)
    _, want2 = _oracle_replay(oracle, open(p).read(), host_in2)
    d_in2, d_out2 = _to_dev(torch, host_in2), torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
    eng.exeOp("ring", d_in2, d_out2, stream)
    eng.waitOp("ring", stream)
    H.assert_bits_equal(d_out2.cpu().numpy().view(np.uint16), want2, "after re-binding")
    # same output tensor, new input only
    eng.exeOp("ring", d_in, d_out2, stream)
    eng.waitOp("ring", stream)
    H.assert_bits_equal(d_out2.cpu().numpy().view(np.uint16), want, "input re-bound alone")


def test_ring_allreduce_in_place_and_back(E, eng, oracle, tmp_path):
    """exeOp with one tensor as input and output (every chunk is read by the op that first writes it, so the
    result is the out-of-place one), then on separate tensors again, then in place again: the executor moves
    the operands where it can and builds the graph again where it cannot."""
    import torch
    p = str(tmp_path / "ring.sched")
    E.write_ring_allreduce(p, "bf16", "sum", 8, 70_001)
    eng.regOp("ring", p)
    info = eng.opInfo("ring")
    n = info["devices"] * info["elems_per_device"]
    stream = torch.cuda.current_stream().cuda_stream
    for round_, seed in enumerate((81, 82, 83, 84)):
        host_in = H.gen("bf16", n, seed, 0)
        _, want = _oracle_replay(oracle, open(p).read(), host_in)
        d_in = _to_dev(torch, host_in)
        if round_ % 2 == 0:
            eng.exeOp("ring", d_in, d_in, stream)
            eng.waitOp("ring", stream)
            H.assert_bits_equal(d_in.cpu().numpy().view(np.uint16), want, "in place, call %d" % round_)
        else:
            d_out = torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
            eng.exeOp("ring", d_in, d_out, stream)
            eng.waitOp("ring", stream)
            H.assert_bits_equal(d_out.cpu().numpy().view(np.uint16), want, "out of place, call %d" % round_)
            H.assert_bits_equal(d_in.cpu().numpy().view(np.uint16), host_in, "input untouched, call %d" % round_)


def test_python_emitted_schedule(E, eng, oracle, tmp_path):
    import torch
    from pccl_amd import lang
    ir, per = lang.small_message_allreduce(n_slices=4, n_extra=9, lo_bytes=256, hi_bytes=8192, dtype="f32", compute="max")
    p = str(tmp_path / "sm.sched")
    ir.save(p, per)
    eng.regOp("sm", p)
    n = 8 * per
    host_in = H.gen("f32", n, 73, 0)
    _, want = _oracle_replay(oracle, open(p).read(), host_in)
    d_in, d_out = _to_dev(torch, host_in), torch.zeros(n * 4, dtype=torch.uint8, device="cuda")
    eng.exeOp("sm", d_in, d_out)
    eng.waitOp("sm")
    H.assert_bits_equal(d_out.cpu().numpy().view(np.float32), want, "python-emitted small-message schedule")


def test_direct_allreduce_8_inputs(E, eng, oracle, tmp_path):
    """NVLS-style: every slice is one 8-input reduce in fixed rank order, then a 7-way broadcast copy."""
    import torch
    p = str(tmp_path / "direct.sched")
    E.write_direct_allreduce(p, "f16", "sum", 8, 4099)
    eng.regOp("direct", p)
    n = 8 * 8 * 4099
    host_in = H.gen("f16", n, 74, 0)
    hdr, want = _oracle_replay(oracle, open(p).read(), host_in)
    d_in, d_out = _to_dev(torch, host_in), torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
    eng.exeOp("direct", d_in, d_out)
    eng.waitOp("direct")
    got = d_out.cpu().numpy().view(np.uint16)
    H.assert_bits_equal(got, want, "direct all-reduce")
    per = hdr["elems_per_device"]
    wide = [host_in[r * per:(r + 1) * per] for r in range(8)]
    H.assert_bits_equal(got[:per], oracle.reduce("f16", "sum", wide), "equals one 8-input fold in rank order")


@pytest.mark.parametrize("own_gather,chunk", [(False, 40_003), (True, 1 << 20)])
def test_rank_share_schedule_through_exeop(E, eng, oracle, tmp_path, own_gather, chunk):
    """One rank's 14 ring steps at world size 8 (7 reduce-copy steps into an output chunk and the one send
    buffer, 7 copy steps) as a schedule file through Engine::regOp / exeOp: 14 ops ordered by the hazards of their
    buffers, which the executor sends to the queue as one launch.  Twice, on fresh inputs, against the CPU
    checker replaying the file."""
    import torch
    from pccl_amd import lang
    ir, per = lang.ring_rank_share(8, chunk, dtype="bf16", gather_buffers_of_their_own=own_gather)
    p = str(tmp_path / "share.sched")
    ir.save(p, per)
    name = "share%d" % own_gather
    eng.regOp(name, p)
    info = eng.opInfo(name)
    assert info["n_ops"] == 14 and info["devices"] == (3 if own_gather else 2) and info["elems_per_device"] == 8 * chunk
    n = info["devices"] * per
    stream = torch.cuda.current_stream().cuda_stream
    for it in range(2):
        host_in = H.gen("bf16", n, 79 + it, 0)
        hdr, want = _oracle_replay(oracle, open(p).read(), host_in)
        d_in, d_out = _to_dev(torch, host_in), torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
        eng.exeOp(name, d_in, d_out, stream)
        eng.waitOp(name, stream)
        got = d_out.cpu().numpy().view(np.uint16)
        H.assert_bits_equal(got[:per], want[:per], "result, run %d" % it)
        H.assert_bits_equal(got[per:per + chunk], want[per:per + chunk], "send buffer, run %d" % it)
        assert not got[per + chunk:].any(), "nothing else of the output tensor is written"
        # the result is the gradient with chunk c replaced: chunks 1..7 hold what the copy steps brought, chunk 0 the last fold
        src = 2 if own_gather else 1
        for s in range(7):
            c = (8 - s) % 8
            H.assert_bits_equal(got[c * chunk:(c + 1) * chunk], host_in[src * per + s * chunk:src * per + (s + 1) * chunk], "copy step %d" % s)


@pytest.mark.parametrize("parts", [1, 4])
def test_signalled_ring_schedule(E, eng, oracle, tmp_path, parts):
    """A schedule whose cross-rank hand-over goes through NOTIFY / GET_NOTIFIED on the workspace's
    signal slots (no dependency edge between ranks), registered from a file and run twice; with one slot per
    signal (format version 1) and with a slot per part of the chunk (version 2)."""
    import torch
    from pccl_amd import lang
    ir, per = lang.ring_allreduce_signalled(8, 2500, dtype="bf16", first_slot=16, signal_parts=parts)
    p = str(tmp_path / "sig.sched")
    ir.save(p, per)
    text = open(p).read()
    assert "NOTIFY" in text and "GET_NOTIFIED" in text and text.startswith("pccl-schedule %d\n" % (1 if parts == 1 else 2))
    eng.regOp("sig", p)
    hdr, ops = S.parse_schedule_text(text)
    n = 8 * per
    for it in range(2):
        host_in = H.gen("bf16", n, 76 + it, 0)
        want = np.zeros(n, dtype=np.uint16)
        bufs = {"in": host_in, "out": want}
        # file order is a valid order (each rank's program order, steps ascending)
        slots = S.replay_with_signals(oracle, ops, range(len(ops)), lambda b, r, e, c: bufs[b][r * per + e:r * per + e + c])
        assert slots == {16 + k: 14 for k in range(8 * parts)}
        d_in, d_out = _to_dev(torch, host_in), torch.zeros(n * 2, dtype=torch.uint8, device="cuda")
        eng.exeOp("sig", d_in, d_out)
        eng.waitOp("sig")
        H.assert_bits_equal(d_out.cpu().numpy().view(np.uint16), want, "signalled ring, run %d" % it)
        for r in range(1, 8):
            H.assert_bits_equal(want[r * per:(r + 1) * per], want[:per], "rank %d equals rank 0" % r)


def test_exe_op_on_another_stream_waits_for_the_run_before(E, eng, oracle, tmp_path):
    """A registered op is one graph on the device and runs one launch at a time: exeOp on a second
    stream, issued while the run on the first may still be going, starts behind it, and each call's
    result is the checker's."""
    import torch
    p = str(tmp_path / "ring2s.sched")
    E.write_ring_allreduce(p, "bf16", "sum", 8, 1 << 19)
    eng.regOp("ring2s", p)
    info = eng.opInfo("ring2s")
    n = info["devices"] * info["elems_per_device"]
    text = open(p).read()
    inputs = [H.gen("bf16", n, 171 + k, 0) for k in range(3)]
    wants = [_oracle_replay(oracle, text, a)[1] for a in inputs]
    d_ins = [_to_dev(torch, a) for a in inputs]
    d_outs = [torch.zeros(n * 2, dtype=torch.uint8, device="cuda") for _ in inputs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for rounds in range(2):
        for k in range(3):                      # streams alternate; inputs and outputs change every call
            eng.exeOp("ring2s", d_ins[k], d_outs[k], streams[k % 2].cuda_stream)
        # the same tensors again on the other stream, without anything in between
        eng.exeOp("ring2s", d_ins[2], d_outs[2], streams[1].cuda_stream)
        eng.waitOp("ring2s", streams[1].cuda_stream)
        torch.cuda.synchronize()
        for k in range(3):
            H.assert_bits_equal(d_outs[k].cpu().numpy().view(np.uint16), wants[k], "round %d, call %d" % (rounds, k))
            d_outs[k].zero_()
        torch.cuda.synchronize()


def test_exe_op_argument_errors(E, eng, tmp_path):
    import torch
    p = str(tmp_path / "r.sched")
    E.write_ring_allreduce(p, "f32", "sum", 2, 64)
    eng.regOp("small", p)
    big, tiny = torch.zeros(256, device="cuda"), torch.zeros(8, device="cuda")
    with pytest.raises(E.EngineError):
        eng.exeOp("small", tiny, big)
    with pytest.raises(E.EngineError):
        eng.exeOp("never_registered", big, big)
    with pytest.raises(E.EngineError):
        eng.regOp("missing", str(tmp_path / "does_not_exist.sched"))


def test_plugin_layer_reduce_copy(E, oracle):
    """Registry names -> HipExecutor::reduceCopy -> C ABI."""
    import torch
    ins = [H.gen("i32", 100001, 75, k) for k in range(4)]
    want = oracle.reduce("i32", "max", ins)
    d_in = [_to_dev(torch, a) for a in ins]
    d_out = torch.zeros(100001 * 4, dtype=torch.uint8, device="cuda")
    E.reduce_copy("i32", "max", d_in, [d_out], 100001, torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    H.assert_bits_equal(d_out.cpu().numpy().view(np.int32), want, "plugin-layer reduce_copy")
    with pytest.raises(E.EngineError):
        E.reduce_copy("c64", "sum", d_in, [d_out], 4)
    p = E.allocate("rocm", 3 << 20)
    assert p and p % 256 == 0
    E.deallocate("rocm", p)
    assert E.allocate("rocm", 0) is None


@pytest.mark.parametrize("dtype,compute", [("f32", "max"), ("f64", "sum"), ("u32", "min"), ("f8e4m3", "sum"), ("f16", "prod")])
def test_ring_schedule_other_dtypes(E, eng, oracle, tmp_path, dtype, compute):
    """The schedule file, engine and queue carry every dtype / compute name the plugin registers."""
    import torch
    p = str(tmp_path / "ring.sched")
    E.write_ring_allreduce(p, dtype, compute, 4, 5001)
    eng.regOp("ring_" + dtype, p)
    info = eng.opInfo("ring_" + dtype)
    assert info["elem_bytes"] == H.ELEM_BYTES[dtype]
    n = info["devices"] * info["elems_per_device"]
    kw = dict(kind="uniform", lo=0.7, hi=1.4) if compute == "prod" else {}
    host_in = H.gen(dtype, n, 75, 0, **kw)
    hdr, want = _oracle_replay(oracle, open(p).read(), host_in)
    d_in = _to_dev(torch, host_in)
    d_out = torch.zeros(n * H.ELEM_BYTES[dtype], dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    eng.exeOp("ring_" + dtype, d_in, d_out, stream)
    eng.waitOp("ring_" + dtype, stream)
    H.assert_bits_equal(d_out.cpu().numpy().view(H.STORAGE[dtype]), want, "engine ring %s %s" % (dtype, compute))


@pytest.mark.parametrize("which", ["reduce_scatter", "all_gather", "direct", "broadcast", "all_to_all"])
def test_python_emitted_collectives(E, eng, oracle, tmp_path, which):
    """The other emitters of pccl_amd.lang through regOp / exeOp, against the CPU replay of the
    same schedule file."""
    import torch
    from pccl_amd import lang
    W, n, dtype = 8, 20011, "bf16"
    ir, per = {"reduce_scatter": lambda: lang.ring_reduce_scatter(W, n, dtype, "sum"),
               "all_gather": lambda: lang.ring_all_gather(W, n, dtype),
               "direct": lambda: lang.direct_allreduce(W, n, dtype, "sum"),
               "broadcast": lambda: lang.broadcast(W, 3 * n, root=5, dtype=dtype),
               "all_to_all": lambda: lang.all_to_all(W, n, dtype)}[which]()
    p = str(tmp_path / (which + ".sched"))
    ir.save(p, per)
    eng.regOp(which, p)
    total = W * per
    host_in = H.gen(dtype, total, 77, 0)
    hdr, want = _oracle_replay(oracle, open(p).read(), host_in)
    d_in, d_out = _to_dev(torch, host_in), torch.zeros(total * 2, dtype=torch.uint8, device="cuda")
    eng.exeOp(which, d_in, d_out)
    eng.waitOp(which)
    H.assert_bits_equal(d_out.cpu().numpy().view(np.uint16), want, which)


def test_schedule_staging_through_the_workspace(E, eng, oracle, tmp_path):
    """Operands named "ws" live in per-device regions of the engine's workspace, laid out by the
    executor (back to back, each on a 256-byte boundary): ws[r] = in[r] + in[r+1]; out[r] = ws[r]."""
    import torch
    W, n = 4, 3 * 1000 * 1000 + 7      # 12 MB per region, a ragged size: the regions' starts are rounded to 256 bytes
    lines = ["pccl-schedule 1", "name staged", "dtype f32", "compute sum", "devices %d" % W,
             "elems_per_device %d" % n, "ops %d" % (2 * W)]
    for r in range(W):
        lines.append("op %d REDUCE %d deps 0 src 2 in %d 0 in %d 0 dst 1 ws %d 0" % (r, n, r, (r + 1) % W, r))
    for r in range(W):
        lines.append("op %d COPY %d deps 1 %d src 1 ws %d 0 dst 1 out %d 0" % (W + r, n, r, r, r))
    p = tmp_path / "staged.sched"
    p.write_text("\n".join(lines) + "\n")
    eng.regOp("staged", str(p))
    host_in = H.gen("f32", W * n, 75, 0)
    d_in, d_out = _to_dev(torch, host_in), torch.zeros(W * n * 4, dtype=torch.uint8, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream
    eng.exeOp("staged", d_in, d_out, stream)
    eng.waitOp("staged", stream)
    got = d_out.cpu().numpy().view(np.float32)
    for r in range(W):
        want = oracle.reduce("f32", "sum", [host_in[r * n:(r + 1) * n], host_in[((r + 1) % W) * n:((r + 1) % W + 1) * n]])
        H.assert_bits_equal(got[r * n:(r + 1) * n], want, "device %d" % r)
    # a region that cannot fit the 256 MiB workspace is refused
    big = (1 << 28) // 4 // W + 4096
    lines[5] = "elems_per_device %d" % big
    lines[7:] = ["op %d REDUCE %d deps 0 src 2 in %d 0 in %d 0 dst 1 ws %d 0" % (r, big, r, (r + 1) % W, r) for r in range(W)] + \
                ["op %d COPY %d deps 1 %d src 1 ws %d 0 dst 1 out %d 0" % (W + r, big, r, r, r) for r in range(W)]
    p2 = tmp_path / "too_big.sched"
    p2.write_text("\n".join(lines) + "\n")
    eng.regOp("too_big", str(p2))
    x = torch.zeros(W * big * 4, dtype=torch.uint8, device="cuda")
    with pytest.raises(E.EngineError):
        eng.exeOp("too_big", x, x.clone(), stream)


def test_extension_module_exeop_on_torch_tensors(E, oracle, tmp_path):
    """The reference's Python entry point: pccl.engine_c.Engine(rank, world).exeOp(name, input, output)
    on torch tensors (csrc/python_api.cc:13-20, include/engine.h:19), here pccl_amd.engine_c: a ring
    all-reduce over 8 virtual ranks in bf16, on torch's current stream, against the CPU checker."""
    import torch
    from pccl_amd import engine_c
    p = str(tmp_path / "ring.sched")
    E.write_ring_allreduce(p, "bf16", "sum", 8, 54321)
    eng = engine_c.Engine(0, 1)
    eng.initEngine()
    eng.regOp("ring", p)
    hdr, _ = S.parse_schedule_text(open(p).read())
    n = hdr["devices"] * hdr["elems_per_device"]
    for it, stream in enumerate((torch.cuda.current_stream(), torch.cuda.Stream())):
        host_in = H.gen("bf16", n, 171 + it, 0)
        _, want = _oracle_replay(oracle, open(p).read(), host_in)
        with torch.cuda.stream(stream):
            x = torch.from_numpy(host_in.view(np.int16)).cuda().view(torch.bfloat16)
            y = torch.zeros(n, dtype=torch.bfloat16, device="cuda")
            eng.exeOp("ring", x, y)
            eng.waitOp("ring")
        got = y.view(torch.int16).cpu().numpy().view(np.uint16)
        H.assert_bits_equal(got, want, "extension module, run %d" % it)
    with pytest.raises(RuntimeError):
        eng.exeOp("ring", x[:100], y)          # too small for the schedule
    with pytest.raises(RuntimeError):
        eng.exeOp("ring", x.cpu(), y)          # not a device tensor
    with pytest.raises(RuntimeError):
        eng.exeOp("unknown", x, y)
    del eng
