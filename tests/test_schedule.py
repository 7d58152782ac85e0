"""The product's schedule classes against the oracle streams, instruction by instruction."""
import json
import os

import pytest

from bamboo_amd import schedule as S
from bamboo_amd.utils import get_redundant_stage_ids, get_redundant_user_stage_ids
from oracle import schedule as osched


def as_tuples(steps):
    out = []
    for cmds in steps:
        row = []
        for c in cmds:
            row.append((c.name, c.kwargs.get("buffer_id"), c.kwargs.get("stage_id")))
        out.append(row)
    return out


@pytest.mark.parametrize("stages,mbs", [(s, m) for s in range(1, 7) for m in range(1, 11)])
def test_train_schedule_equals_oracle(stages, mbs):
    for sid in range(stages):
        got = as_tuples(S.TrainSchedule(micro_batches=mbs, stages=stages, stage_id=sid))
        assert got == osched.train_schedule(mbs, stages, sid)


@pytest.mark.parametrize("stages,mbs", [(2, 3), (4, 4), (4, 8), (4, 16), (5, 7), (6, 10)])
def test_eager_and_failover_equal_oracle(stages, mbs):
    for sid in range(stages - 1):
        mk = lambda s: S.TrainSchedule(micro_batches=mbs, stages=stages, stage_id=s)
        eager = as_tuples(S.EagerRecoverySchedule(mk(sid), mk(sid + 1)))
        own, nxt = osched.train_schedule(mbs, stages, sid), osched.train_schedule(mbs, stages, sid + 1)
        assert eager == osched.eager_merge(own, nxt)
        T = len(own)
        for fs, cs in [(0, 0), (T // 3, T // 3), (T // 3, T // 2), (T - 1, T - 1), (0, T // 2)]:
            got = as_tuples(S.NextStageFailoverSchedule(mk(sid), mk(sid + 1), failed_step=fs, curr_step=cs))
            assert got == osched.next_stage_failover(own, nxt, fs, cs)


@pytest.mark.parametrize("stages,mbs", [(3, 3), (4, 4), (4, 8), (5, 7)])
def test_prev_stage_and_allreduce_failover_equal_oracle(stages, mbs):
    mk = lambda s: S.TrainSchedule(micro_batches=mbs, stages=stages, stage_id=s)
    for sid in range(2, stages):                  # the stage after a lost middle stage
        own = osched.train_schedule(mbs, stages, sid)
        eager_own = osched.eager_merge(own, osched.train_schedule(mbs, stages, (sid + 1) % stages))
        T = len(own)
        for fs, cs in [(0, 0), (T // 3, T // 3), (T // 3, T // 2), (T // 2, T - 1)]:
            got = as_tuples(S.PrevStageFailoverSchedule(mk(sid - 1), mk(sid), failed_step=fs, curr_step=cs))
            want = osched.prev_stage_failover(own, fs, cs)
            assert got == want
            # what the definition fixes: before curr_step nothing but gradient re-sends, every own
            # gradient send of the steps before failed_step exactly once, afterwards the own stream
            resent = [c for i, cmds in enumerate(want) if i < cs for c in cmds]
            assert all(c[0] == "SendGrad" for c in resent)
            assert resent == [c for i, cmds in enumerate(own) if i < min(fs, cs) for c in cmds if c[0] == "SendGrad"]
            assert want[cs:] == own[cs:]
            # wrapped around the stage's own RC stream, as the engine builds it
            wrapped = as_tuples(S.PrevStageFailoverSchedule(
                mk(sid - 1), S.EagerRecoverySchedule(mk(sid), mk((sid + 1) % stages)), failed_step=fs, curr_step=cs))
            assert wrapped == osched.prev_stage_failover(eager_own, fs, cs)
        for fs in (0, T // 2, T):
            got = as_tuples(S.AllReduceFailoverSchedule(mk(sid), [[] for _ in range(T)], failed_step=fs))
            assert got == osched.allreduce_failover(own, fs)


def test_upstream_invariants():
    """tests/unit/test_pipe_schedule.py:126-157 of the reference tree, on this implementation."""
    sched = S.TrainSchedule(stages=3, micro_batches=4, stage_id=0)
    assert sched.num_micro_batches == 4
    full = list(iter(sched))
    for cmds in full:
        for c in cmds:
            assert not isinstance(c, (S.SendGrad, S.RecvActivation))
            if isinstance(c, S.BufferOpInstruction):
                assert 0 <= c.buffer_id < sched.num_pipe_buffers()
    sched = S.TrainSchedule(stages=3, micro_batches=4, stage_id=2)
    for cmds in sched:
        for c in cmds:
            assert not isinstance(c, (S.SendActivation, S.RecvGrad))
    sched = S.TrainSchedule(stages=3, micro_batches=4, stage_id=1)
    assert sched.stage == 1 and sched.num_stages == 3 and not sched.is_first_stage and not sched.is_last_stage


def test_repr_and_call_to_str():
    # tests/unit/test_runtime_utils.py:14-22 of the reference tree
    golden = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_known_answers.json")
    for c in json.load(open(golden))["call_to_str"]["cases"]:
        assert S.call_to_str(*c["args"], **c["kwargs"]) == c["out"]
    assert repr(S.ForwardPass(2, 1)) == "ForwardPass(buffer_id=2, stage_id=1)"
    assert repr(S.OptimizerStep()) == "OptimizerStep()"


def test_lazy_schedule_pings():
    mk = lambda s: S.TrainSchedule(micro_batches=4, stages=4, stage_id=s)
    lazy = list(S.LazyRecoverySchedule(mk(1), mk(2)))
    plain = list(mk(1))
    assert len(lazy) == len(plain)
    for t, (a, b) in enumerate(zip(lazy, plain)):
        extra = [c for c in a if getattr(c, "buffer_id", 0) == -1]
        assert [c for c in a if getattr(c, "buffer_id", 0) != -1] == b
        talks = any(isinstance(c, S.CommunicationInstruction) for c in b)
        first_half = t < 4 + 4 - 1
        assert len(extra) == (0 if talks or not first_half else 1)


@pytest.mark.parametrize("stages,mbs", [(s, m) for s in range(2, 7) for m in range(1, 11)])
def test_lazy_schedule_equals_oracle(stages, mbs):
    """First, middle and last stage branches of LazyRecoverySchedule (reference schedule.py:483-501)."""
    for sid in range(stages):
        mk = lambda s: S.TrainSchedule(micro_batches=mbs, stages=stages, stage_id=s)
        got = as_tuples(S.LazyRecoverySchedule(mk(sid), mk((sid + 1) % stages)))
        assert got == osched.lazy_merge(osched.train_schedule(mbs, stages, sid), mbs, stages, sid)


def test_redundancy_helpers():
    for level in (0, 1):
        for stages in range(1, 6):
            for sid in range(stages):
                assert get_redundant_stage_ids(level, sid, stages) == osched.redundant_stage_ids(level, sid, stages)
                assert get_redundant_user_stage_ids(level, sid, stages) == osched.redundant_user_stage_ids(level, sid, stages)
