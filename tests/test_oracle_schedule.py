"""Pins of the schedule oracle: closed forms vs. the piecewise parity rules, the invariants of
the upstream unit test (tests/unit/test_pipe_schedule.py:126-157 of the reference tree), brute
force over small (S, M), and the hand trace S=4, M=4, stage 1."""
import itertools

import pytest

from oracle import schedule as osched


def piecewise(stages, stage_id, step_id):
    """The four parity cases written out literally (reference schedule.py:6-46)."""
    even = lambda x: x % 2 == 0
    if even(step_id) and even(stage_id):
        return step_id // 2 - stage_id // 2, True
    if not even(step_id) and not even(stage_id):
        return (step_id - 1) // 2 - stage_id // 2, True
    if even(step_id) and not even(stage_id):
        return step_id // 2 - stages + (stage_id + 1) // 2, False
    return (step_id - 1) // 2 - stages + 1 + stage_id // 2, False


def test_closed_form_matches_piecewise():
    for S in range(1, 9):
        for s in range(S):
            for t in range(0, 2 * (12 + S)):
                assert osched.step_to_micro_batch(S, s, t) == piecewise(S, s, t)


@pytest.mark.parametrize("S,M", [(S, M) for S in range(1, 7) for M in range(1, 11)])
def test_train_schedule_invariants(S, M):
    streams = [osched.train_schedule(M, S, s) for s in range(S)]
    for s, steps in enumerate(streams):
        assert len(steps) == 2 * (M + S - 1)
        flat = [c for cmds in steps for c in cmds]
        kinds = [c[0] for c in flat]
        if s == 0:
            assert "SendGrad" not in kinds and "RecvActivation" not in kinds
        if s == S - 1:
            assert "SendActivation" not in kinds and "RecvGrad" not in kinds
        for name, k, sid in flat:
            if k is not None:
                assert 0 <= k < M
        # every micro-batch: exactly one forward, one backward, forward first; one compute per step
        pos_f, pos_b = {}, {}
        for t, cmds in enumerate(steps):
            comp = [c for c in cmds if c[0] in ("ForwardPass", "BackwardPass")]
            assert len(comp) <= 1
            for name, k, _ in comp:
                (pos_f if name == "ForwardPass" else pos_b).setdefault(k, []).append(t)
        assert sorted(pos_f) == list(range(M)) and sorted(pos_b) == list(range(M))
        for k in range(M):
            assert len(pos_f[k]) == 1 and len(pos_b[k]) == 1 and pos_f[k][0] < pos_b[k][0]
        assert steps[-1][-2:] == [("ReduceGrads", None, s), ("OptimizerStep", None, None)]
        loads = [c for c in flat if c[0] == "LoadMicroBatch"]
        assert len(loads) == (M if s in (0, S - 1) else 0)
    # pairing: a send on stage s and the matching recv on the neighbour land in the same step
    for s in range(S - 1):
        for t in range(2 * (M + S - 1)):
            sa = [c[1] for c in streams[s][t] if c[0] == "SendActivation"]
            ra = [c[1] for c in streams[s + 1][t] if c[0] == "RecvActivation"]
            assert sa == ra
            rg = [c[1] for c in streams[s][t] if c[0] == "RecvGrad"]
            sg = [c[1] for c in streams[s + 1][t] if c[0] == "SendGrad"]
            assert rg == sg


def _short(cmds):
    ab = {"RecvActivation": "RA", "SendActivation": "SA", "RecvGrad": "RG", "SendGrad": "SG",
          "ForwardPass": "F", "BackwardPass": "B", "ReduceGrads": "Red", "OptimizerStep": "Opt",
          "LoadMicroBatch": "L"}
    return [f"{ab[n]}{'' if k is None else k}{'' if s in (None, 1) else '@' + str(s)}" for n, k, s in cmds]


HAND_TRACE = [  # S=4, M=4, own stage 1, shadow stage 2 (commands of stage 2 carry @2)
    [], ["RA0", "F0"], ["SA0"], ["RA1", "F1"], ["SA1"], ["RA2", "F2"],
    ["RA0@2", "F0@2", "SA2", "RG0", "B0"], ["RA3", "SG0", "F3"],
    ["RA1@2", "F1@2", "SA3", "RG1", "B1"], ["SG1"],
    ["RA2@2", "F2@2", "RG2", "B2"], ["SG2"],
    ["RA3@2", "F3@2", "RG3", "B3"], ["SG3", "Red", "Opt"],
]


def test_hand_trace_eager():
    own = osched.train_schedule(4, 4, 1)
    nxt = osched.train_schedule(4, 4, 2)
    merged = osched.eager_merge(own, nxt)
    assert [_short(c) for c in merged] == HAND_TRACE
    plain = [[x for x in step if "@2" not in x] for step in HAND_TRACE]
    assert [_short(c) for c in own] == plain


@pytest.mark.parametrize("S,M", [(S, M) for S in range(2, 7) for M in range(1, 11)])
def test_eager_invariants(S, M):
    for s in range(S - 1):
        r = s + 1
        merged = osched.eager_merge(osched.train_schedule(M, S, s), osched.train_schedule(M, S, r))
        rc_f = [(t, c[1]) for t, cmds in enumerate(merged) for c in cmds if c[0] == "ForwardPass" and c[2] == r]
        assert [k for _, k in rc_f] == list(range(M))       # exactly M redundant forwards, in order
        for t, k in rc_f:
            names = [(c[0], c[1], c[2]) for c in merged[t]]
            i_rc = names.index(("ForwardPass", k, r))
            i_rg = names.index(("RecvGrad", k, s))           # same step, directly before the own RecvGrad(k)
            assert i_rc < i_rg
            # the input of the redundant forward is the own output of the same micro-batch
            own_f = [tt for tt, cmds in enumerate(merged) for c in cmds if c == ("ForwardPass", k, s)]
            assert own_f[0] < t
    # last stage: its successor (wrap-around stage 0) is never computed redundantly
    last = osched.eager_merge(osched.train_schedule(M, S, S - 1), osched.train_schedule(M, S, 0))
    assert not any(c[0] == "ForwardPass" and c[2] == 0 for cmds in last for c in cmds)


@pytest.mark.parametrize("S,M", [(3, 4), (4, 4), (4, 8), (5, 6)])
def test_failover_structure(S, M):
    for s in range(S - 1):
        own, nxt = osched.train_schedule(M, S, s), osched.train_schedule(M, S, s + 1)
        T = len(own)
        for cut in range(0, T):
            merged = osched.next_stage_failover(own, nxt, cut, cut)
            flat = [c for cmds in merged[cut:] for c in cmds]
            # no own<->successor transfer is left after the merge point
            assert ("SendActivation" not in [c[0] for c in flat if c[2] == s])
            assert ("SendGrad" not in [c[0] for c in flat if c[2] == s + 1])
            kinds = [c[0] for c in flat]
            assert kinds.count("OptimizerStep") == 1 and kinds.count("ReduceGrads") == 2
            # replayed part: only the successor's commands, without its sends
            for cmds in merged[:cut]:
                assert all(c[2] == s + 1 or c[0] == "LoadMicroBatch" for c in cmds)
                assert not any(c[0] in ("SendActivation", "SendGrad") for c in cmds)
            # every successor backward appears exactly once over replay + merge
            b = [c[1] for cmds in merged for c in cmds if c[0] == "BackwardPass" and c[2] == s + 1]
            assert sorted(b) == list(range(M))


def test_worked_failover_step():
    """S=4, M=4, own stage 1, step 6 (plain streams on both sides)."""
    own, nxt = osched.train_schedule(4, 4, 1), osched.train_schedule(4, 4, 2)
    merged = osched.next_stage_failover(own, nxt, 0, 0)
    assert merged[6] == [("RecvActivation", 2, 2), ("RecvGrad", 0, 1), ("BackwardPass", 0, 1), ("ForwardPass", 2, 2)]


def test_redundancy_ids():
    assert osched.redundant_stage_ids(0, 1, 4) == []
    assert osched.redundant_stage_ids(1, 1, 4) == [2]
    assert osched.redundant_stage_ids(1, 3, 4) == [0]
    assert osched.redundant_user_stage_ids(1, 2, 4) == [1]
    assert osched.redundant_user_stage_ids(1, 0, 4) == [3]


def test_lazy_merge_hand_trace():
    """S = 4, M = 2, worked by hand from the three branches of the reference
    (schedule.py:483-501).  T = 10 steps, first half = steps 0..4.  L = RecvActivation(-1), C = SendActivation(-1);
    a stage's forward steps are those of its own parity.
      stage 0: L on steps 0, 2, 4, 6, 8 (every forward step, valid micro-batch or not)
      stage 1: quiet steps of the first half are 0 (backward parity -> C) only (1..4 carry transfers)
      stage 2: quiet steps 0 (forward parity -> L) and 1 (-> C)
      stage 3: L on quiet forward steps of the first half: 1 (3 carries RecvActivation(0));
               C on every step with stage 0's forward parity: 0, 2, 4, 6, 8, in front of everything else"""
    M, S = 2, 4
    pings = {}
    for s in range(S):
        steps = osched.lazy_merge(osched.train_schedule(M, S, s), M, S, s)
        pings[s] = {i: [c[0][0] for c in cmds if c[1] == -1] for i, cmds in enumerate(steps) if any(c[1] == -1 for c in cmds)}
        # nothing but pings is added, and pings come first
        for got, own in zip(steps, osched.train_schedule(M, S, s)):
            assert [c for c in got if c[1] != -1] == own
            n = sum(1 for c in got if c[1] == -1)
            assert all(c[1] == -1 for c in got[:n])
    assert pings[0] == {0: ["R"], 2: ["R"], 4: ["R"], 6: ["R"], 8: ["R"]}
    assert pings[1] == {0: ["S"]}
    assert pings[2] == {0: ["R"], 1: ["S"]}
    assert pings[3] == {0: ["S"], 1: ["R"], 2: ["S"], 4: ["S"], 6: ["S"], 8: ["S"]}


@pytest.mark.parametrize("S,M", [(S, M) for S in range(2, 7) for M in range(1, 11) if M >= S - 1])
def test_lazy_pings_pair_up_around_the_ring(S, M):
    """A one-element send is a blocking transfer: whenever stage s calls its successor, the successor (the
    first stage for the last one) listens in the same step, and nobody listens without a caller.  Holds from
    M >= S - 1 on (with fewer micro-batches the reference's own rule leaves a few pings unanswered)."""
    streams = [osched.lazy_merge(osched.train_schedule(M, S, s), M, S, s) for s in range(S)]
    for i in range(osched.total_steps(M, S)):
        for s in range(S):
            calls = [c for c in streams[s][i] if c[:2] == ("SendActivation", -1)]
            listens = [c for c in streams[(s + 1) % S][i] if c[:2] == ("RecvActivation", -1)]
            assert len(calls) == len(listens) <= 1, (i, s)
