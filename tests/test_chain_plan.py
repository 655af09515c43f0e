"""The executor's chain plan (pccl_hip_plan_chains, host only): which ops run behind each other in one
workgroup, and which chains may run in one pass with the value kept in registers.  No GPU needed:
operands are plain numbers that stand for device addresses."""
import pytest

from pccl_amd import hip

ES = 4  # f32


def op(ins, outs, deps, count=1000, dtype="f32", compute="sum"):
    return dict(dtype=dtype, compute=compute, ins=[a for a in ins], outs=[a for a in outs], count=count, deps=list(deps))


def buf(k, n=1000):
    """Address of buffer k: buffers are far enough apart not to overlap."""
    return 0x100000 + k * (n * 16 + 4096)


def test_single_predecessor_and_successor_make_a_chain():
    a, b, c, t, u, v = (buf(k) for k in range(6))
    ops = [op([a, b], [t], []), op([t, c], [u], [0]), op([u], [v], [1])]
    plan = hip.plan_chains(ops, [1, 1, 1], ES)
    assert [p[0] for p in plan] == [1, 2, -1]           # 0 -> 1 -> 2
    assert plan[0][1] == 3 and plan[1][1] == 1 and plan[2][1] == 1
    assert plan[0][2] == 1 and plan[0][3] == 0          # one pass, rows from 0
    assert plan[1][2] == 0                              # the handed-on value is input 0 of op 1
    # ... input 1 when the operands are the other way round
    ops[1] = op([c, t], [u], [0])
    assert hip.plan_chains(ops, [1, 1, 1], ES)[1][2] == 1


def test_no_chain_across_a_fan_out_or_a_fan_in():
    a, b, c, t, u, v, w = (buf(k) for k in range(7))
    fan_out = [op([a, b], [t], []), op([t, c], [u], [0]), op([t], [v], [0])]
    assert [p[0] for p in hip.plan_chains(fan_out, [1, 1, 1], ES)] == [-1, -1, -1]
    fan_in = [op([a, b], [t], []), op([a, c], [u], []), op([t, u], [v], [0, 1]), op([v], [w], [2])]
    plan = hip.plan_chains(fan_in, [1, 1, 1, 1], ES)
    assert [p[0] for p in plan] == [-1, -1, 3, -1]      # only 2 -> 3
    assert plan[2][1] == 2 and plan[2][2] == 1


def test_ops_cut_differently_or_of_other_length_do_not_chain():
    a, b, c, t, u = (buf(k, 100000) for k in range(5))
    ops = [op([a, b], [t], [], count=100000), op([t, c], [u], [0], count=100000)]
    assert hip.plan_chains(ops, [4, 4], ES)[0][0] == 1
    assert hip.plan_chains(ops, [4, 5], ES)[0][0] == -1
    ops[1] = op([t, c], [u], [0], count=99999)
    assert hip.plan_chains(ops, [4, 4], ES)[0][0] == -1


def test_many_part_ops_chain_only_where_part_p_needs_part_p():
    n = 100000
    a, b, c, t, u = (buf(k, n) for k in range(5))
    lined_up = [op([a, b], [t], [], count=n), op([t, c], [u], [0], count=n)]
    assert hip.classify_dependencies(lined_up, [8, 8]) == [1]
    assert hip.plan_chains(lined_up, [8, 8], ES)[0][0] == 1
    shifted = [op([a, b], [t], [], count=n), op([t + 64 * ES, c], [u], [0], count=n)]   # reads t 64 elements further on
    assert hip.classify_dependencies(shifted, [8, 8]) == [0]
    assert hip.plan_chains(shifted, [8, 8], ES)[0][0] == -1
    # with one part each the whole op is done before the next starts: a chain again, but through memory
    plan = hip.plan_chains(shifted, [1, 1], ES)
    assert plan[0][0] == 1 and plan[0][2] == 0


def test_one_pass_needs_the_predecessors_output_as_an_input_and_no_other_look_at_the_chain():
    a, b, c, t, u, v = (buf(k) for k in range(6))
    # op 2 reads t again, which the chain wrote: through memory
    ops = [op([a, b], [t], []), op([t, c], [u], [0]), op([u, t], [v], [1])]
    plan = hip.plan_chains(ops, [1, 1, 1], ES)
    assert [p[0] for p in plan] == [1, 2, -1] and plan[0][2] == 0
    # op 1 does not read op 0's output at all (ordered behind it for another reason): through memory
    ops = [op([a, b], [t], []), op([c, a], [u], [0])]
    plan = hip.plan_chains(ops, [1, 1], ES)
    assert plan[0][0] == 1 and plan[0][2] == 0
    # the handed-on value must be OUTPUT 0 of the predecessor
    ops = [op([a, b], [t, v], []), op([v, c], [u], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][2] == 0
    ops = [op([a, b], [v, t], []), op([v, c], [u], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][2] == 1
    # in place on the first op's own input is fine (read before written, pack by pack) ...
    ops = [op([a, b], [a], []), op([a, c], [u], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][2] == 1
    # ... a later op writing over the first op's input is not
    ops = [op([a, b], [t], []), op([t, c], [a], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][2] == 0


def test_a_copy_of_the_previous_ops_output_folds_into_that_op_in_a_chain_through_memory():
    """8 -> 1 followed by the copy 1 -> 7 of its result (a slice of a one-exchange all-reduce): the chain cannot
    run in one pass (eight inputs), so it goes through memory, and the copy is marked as folded (third word 2):
    the fold stores the copy's outputs itself.  Not when the outputs would not fit one op, overlap an operand of
    the fold at a shift, or the copy reads another output than output 0."""
    ins = [buf(k) for k in range(8)]
    t = buf(8)
    outs = [buf(9 + k) for k in range(7)]
    ops = [op(ins, [t], []), op([t], outs, [0])]
    plan = hip.plan_chains(ops, [1, 1], ES)
    assert plan[0][0] == 1 and plan[0][1] == 2 and plan[0][2] == 0 and plan[1][2] == 2
    # too many outputs for one op (2 + 7 > 8)
    ops = [op(ins, [t, buf(20)], []), op([t], outs, [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[1][2] == 0
    # a copy output overlapping an input of the fold 16 elements further on
    ops = [op(ins, [t], []), op([t], [ins[3] + 16 * ES], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[1][2] == 0
    # ... at the same address it is the in-place case, pack by pack: folded
    ops = [op(ins, [t], []), op([t], [ins[3]], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[1][2] == 2
    # the copy reads output 1, not output 0
    ops = [op(ins, [buf(20), t], []), op([t], outs, [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[1][2] == 0
    # a second copy behind a folded one runs by itself (its source is not the op before it that runs), a third folds again
    u, v, w = buf(30), buf(31), buf(32)
    ops = [op(ins, [t], []), op([t], [u], [0]), op([u], [v], [1]), op([v], [w], [2])]
    plan = hip.plan_chains(ops, [1, 1, 1, 1], ES)
    assert [p[0] for p in plan] == [1, 2, 3, -1] and [p[2] for p in plan] == [0, 2, 0, 2]
    # many parts: folded where part p of the copy needs only part p of the fold
    n = 100000
    big = [buf(k, n) for k in range(12)]
    ops = [op(big[:3], [big[3]], [], count=n), op([big[3]], big[4:6], [0], count=n)]
    assert hip.plan_chains(ops, [8, 8], ES)[1][2] == 2
    # (a two-input first op with such a copy behind it runs in one pass instead: nothing to fold)
    ops = [op(big[:2], [big[3]], [], count=n), op([big[3]], big[4:6], [0], count=n)]
    plan = hip.plan_chains(ops, [8, 8], ES)
    assert plan[0][2] == 1 and plan[1][2] == 0


def test_outputs_of_a_one_pass_chain_may_coincide_but_not_overlap_at_a_shift():
    a, b, c, t, u = (buf(k) for k in range(5))
    same = [op([a, b], [t], []), op([t, c], [u], [0]), op([u], [t], [1])]          # writes t again, same address
    assert hip.plan_chains(same, [1, 1, 1], ES)[0][1:3] == (3, 1)
    shifted = [op([a, b], [t], []), op([t, c], [u], [0]), op([u], [t + 64], [1])]  # overlaps t 64 bytes on
    assert hip.plan_chains(shifted, [1, 1, 1], ES)[0][1:3] == (3, 0)
    apart = [op([a, b], [t], []), op([t, c], [u], [0]), op([u], [t + 1000 * ES], [1])]  # just behind t
    assert hip.plan_chains(apart, [1, 1, 1], ES)[0][1:3] == (3, 1)


def test_one_pass_limits():
    bufs = [buf(k) for k in range(64)]
    chain = lambda n: [op([bufs[k], bufs[40]], [bufs[k + 1]], [k - 1] if k else []) for k in range(n)]
    assert hip.plan_chains(chain(16), [1] * 16, ES)[0][1:3] == (16, 1)
    assert hip.plan_chains(chain(17), [1] * 17, ES)[0][1:3] == (17, 0)   # more ops than one pass holds
    # first op with more than two inputs
    ops = [op(bufs[:3], [bufs[10]], []), op([bufs[10], bufs[4]], [bufs[11]], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][1:3] == (2, 0)
    # more than two outputs somewhere
    ops = [op(bufs[:2], [bufs[10]], []), op([bufs[10]], bufs[11:14], [0])]
    assert hip.plan_chains(ops, [1, 1], ES)[0][1:3] == (2, 0)
    # no one-pass code in the kernel instance (forward_elem_bytes 0), or of another element size
    assert hip.plan_chains(chain(3), [1] * 3, 0)[0][1:3] == (3, 0)
    assert hip.plan_chains(chain(3), [1] * 3, 2)[0][1:3] == (3, 0)


def test_rows_of_the_operand_table_follow_the_chains_in_op_order():
    bufs = [buf(k) for k in range(40)]
    # chain A: ops 0 -> 3 -> 5; chain B: ops 1 -> 2; single op 4
    ops = [op([bufs[0], bufs[1]], [bufs[10]], []),
           op([bufs[2], bufs[3]], [bufs[11]], []),
           op([bufs[11], bufs[4]], [bufs[12]], [1]),
           op([bufs[10], bufs[5]], [bufs[13]], [0]),
           op([bufs[6]], [bufs[14]], []),
           op([bufs[13]], [bufs[15]], [3])]
    plan = hip.plan_chains(ops, [1] * 6, ES)
    assert [p[0] for p in plan] == [3, 2, -1, 5, -1, -1]
    assert plan[0][1:] == (3, 1, 0) and plan[1][1:] == (2, 1, 3)
    assert plan[4][1] == 1


def test_signal_ops_do_not_chain():
    a, b, t, u = (buf(k) for k in range(4))
    sig = 0x900000
    ops = [op([a, b], [t], []), dict(primitive=2, signal=sig, value=1, deps=[0]),
           dict(primitive=3, signal=sig + 4, value=1, deps=[]), op([t], [u], [2])]
    assert [p[0] for p in hip.plan_chains(ops, [1, 1, 1, 1], ES)] == [-1, -1, -1, -1]


def test_bad_arguments_are_refused():
    a, b, t = (buf(k) for k in range(3))
    with pytest.raises(hip.PcclError):
        hip.plan_chains([op([a, b], [t], [5])], [1], ES)      # dependency on an op that does not exist
    with pytest.raises(hip.PcclError):
        hip.plan_chains([op([a, b], [t], [])], [0], ES)       # no parts


# ---- which signal ops ride on data ops (pccl_hip_plan_signals, host only) --------------------

def notify(word, value, deps, parts=0):
    return dict(primitive=2, signal=word, value=value, deps=list(deps), parts=parts)


def get_notified(word, value, deps, parts=0):
    return dict(primitive=3, signal=word, value=value, deps=list(deps), parts=parts)


def test_a_ring_step_carries_its_wait_and_its_notify():
    a, b, t, u = (buf(k) for k in range(4))
    sig = 0x900000
    # rank-style sequence: GET -> data -> NOTIFY -> GET -> data -> NOTIFY
    ops = [get_notified(sig, 1, []), op([a, b], [t], [0]), notify(sig + 4, 1, [1]),
           get_notified(sig, 2, [2]), op([t], [u], [3]), notify(sig + 4, 2, [4])]
    assert hip.plan_signals(ops) == [1, -1, 1, 4, -1, 4]
    # the plan looks at kinds and dependency lists only: other addresses, same plan
    moved = [dict(o) for o in ops]
    moved[1] = op([b, a], [u], [0])
    assert hip.plan_signals(moved) == [1, -1, 1, 4, -1, 4]


def test_signals_of_a_word_per_part_cut_their_data_op():
    """A NOTIFY / GET_NOTIFIED of K words (one per part of the data) rides on a data op like a one-word one, and the
    op is then cut into K parts; an op carries such signals of ONE K only."""
    a, b, t, u = (buf(k) for k in range(4))
    sig = 0x900000
    ops = [get_notified(sig, 1, [], parts=8), op([a, b], [t], [0]), notify(sig + 64, 1, [1], parts=8),
           get_notified(sig, 2, [2], parts=8), op([t], [u], [3]), notify(sig + 64, 2, [4], parts=8)]
    assert hip.plan_signals(ops, with_parts=True) == ([1, -1, 1, 4, -1, 4], [8, 8, 8, 8, 8, 8])
    # one word (parts 0 or 1) is the form there always was: carried, the op's cut is the executor's
    plain = [dict(o, parts=1) if "parts" in o else o for o in ops]
    assert hip.plan_signals(plain, with_parts=True) == ([1, -1, 1, 4, -1, 4], [0] * 6)
    # a wait of 8 words and a notify of 4 on one op: the notify comes first in the rule and is carried, the wait stays
    mixed = [get_notified(sig, 1, [], parts=8), op([a, b], [t], [0]), notify(sig + 64, 1, [1], parts=4)]
    assert hip.plan_signals(mixed, with_parts=True) == ([-1, -1, 1], [0, 4, 4])
    # ... a one-word signal beside a per-part one is no conflict
    mixed = [get_notified(sig, 1, []), op([a, b], [t], [0]), notify(sig + 64, 1, [1], parts=4)]
    assert hip.plan_signals(mixed, with_parts=True) == ([1, -1, 1], [0, 4, 4])
    # a per-part signal that no data op can carry (two ops behind it) stays an op of its own
    alone = [op([a], [t], []), op([b], [u], []), notify(sig, 1, [0, 1], parts=16)]
    assert hip.plan_signals(alone, with_parts=True) == ([-1, -1, -1], [0, 0, 0])


def test_signal_ops_that_stay_ops_of_their_own():
    a, b, t, u, v, w = (buf(k) for k in range(6))
    sig = 0x900000
    ops = [op([a, b], [t], []),                 # 0
           op([a, b], [u], []),                 # 1
           notify(sig, 3, [0, 1]),              # 2: behind two ops
           notify(sig + 4, 4, [0]),             # 3: rides on op 0
           notify(sig + 8, 5, [0]),             # 4: op 0 carries one already
           get_notified(sig, 3, []),            # 5: two ops wait for it
           op([t], [v], [5]),                   # 6
           op([u], [w], [5]),                   # 7
           get_notified(sig + 8, 5, []),        # 8: in front of a NOTIFY, not of a data op
           notify(sig + 12, 6, [8]),            # 9: behind a GET_NOTIFIED, not a data op
           get_notified(sig + 12, 6, [])]       # 10: nothing waits for it
    assert hip.plan_signals(ops) == [-1, -1, -1, 0, -1, -1, -1, -1, -1, -1, -1]
    # one data op can carry a wait and a notify at once, but not two waits
    ops = [get_notified(sig, 1, []), get_notified(sig + 4, 1, []), op([a], [t], [0, 1]), notify(sig + 8, 1, [2])]
    assert hip.plan_signals(ops) == [2, -1, -1, 2]


def test_plan_signals_refuses_bad_lists():
    a, t = buf(0), buf(1)
    with pytest.raises(hip.PcclError) as e:
        hip.plan_signals([op([a], [t], [3])])
    assert e.value.code == hip.ERR_GRAPH
    assert hip.plan_signals([]) == []


def _model_plan_signals(ops):
    """The documented rule, restated: NOTIFYs first, in op order (one data op behind it alone, which
    carries none yet); what depended on a carried NOTIFY then depends on its data op; then
    GET_NOTIFIEDs in op order (one data op alone depends on it, which carries no wait yet)."""
    n = len(ops)
    kind = [o.get("primitive", 0) for o in ops]
    deps = [list(o["deps"]) for o in ops]
    data = lambda i: kind[i] < 2
    carrier = [-1] * n
    has_notify, has_wait = set(), set()
    stands_for = list(range(n))
    for v in range(n):
        if kind[v] == 2 and len(deps[v]) == 1 and data(deps[v][0]) and deps[v][0] not in has_notify:
            a = deps[v][0]
            has_notify.add(a)
            carrier[v] = a
            stands_for[v] = a
            deps[v] = []
    deps = [sorted(set(stands_for[d] for d in ds)) for ds in deps]
    succ = [[] for _ in range(n)]
    for i in range(n):
        for d in deps[i]:
            succ[d].append(i)
    for v in range(n):
        if kind[v] == 3 and len(succ[v]) == 1 and data(succ[v][0]) and succ[v][0] not in has_wait:
            b = succ[v][0]
            has_wait.add(b)
            carrier[v] = b
    return carrier


def test_plan_signals_follows_the_documented_rule_on_random_programs():
    import random
    rng = random.Random(31)
    carried = 0
    for case in range(400):
        n = rng.randint(1, 24)
        ops = []
        for i in range(n):
            k = min(i, rng.choice([0, 1, 1, 1, 2, 3]))
            deps = rng.sample(range(i), k)
            r = rng.random()
            if r < 0.5:
                ops.append(op([buf(2 * i)], [buf(2 * i + 1)], deps))
            elif r < 0.75:
                ops.append(notify(0x900000 + 4 * rng.randint(0, 5), rng.randint(1, 9), deps))
            else:
                ops.append(get_notified(0x900000 + 4 * rng.randint(0, 5), rng.randint(1, 9), deps))
        got = hip.plan_signals(ops)
        assert got == _model_plan_signals(ops), "case %d: %r" % (case, ops)
        carried += sum(1 for c in got if c >= 0)
        for v, c in enumerate(got):
            if c >= 0:
                assert ops[v].get("primitive", 0) >= 2 and ops[c].get("primitive", 0) < 2
    assert carried > 300
