"""Instruction streams that drive one pipeline stage.

Same names, constructor arguments and step-by-step output as the reference's
``deepspeed/runtime/pipe/schedule.py`` (instruction classes :552-732, ``TrainSchedule``
:225-310, ``ResilientPipeSchedule`` and its subclasses :313-524), so that code written
against the reference engine (``for step_cmds in sched: for cmd in step_cmds: ...``) runs
unchanged.  The implementation is table driven: a 1F1B step is a forward step when step
and stage have the same parity, its micro-batch is ``(t - s) / 2``; otherwise it is a
backward step of micro-batch ``(t + s + 1) / 2 - S``.
"""
from abc import ABC, abstractmethod


def call_to_str(base, *args, **kwargs):
    """``name(arg, key=value)`` rendering used for instruction reprs
    (reference: deepspeed/runtime/utils.py:733-752)."""
    parts = [repr(a) for a in args] + [f"{k}={v!r}" for k, v in kwargs.items()]
    return f"{base}({', '.join(parts)})"


# ------------------------------------------------------------------------------ instructions
class PipeInstruction:
    """Keyword arguments become attributes; ``kwargs`` keeps them for dispatch."""

    def __init__(self, **kwargs):
        self.name = type(self).__name__
        self.kwargs = kwargs
        self.__dict__.update(kwargs)

    def __repr__(self):
        return call_to_str(self.name, **self.kwargs)

    def __eq__(self, other):
        return type(self) is type(other) and self.kwargs == other.kwargs

    def __hash__(self):
        return hash((self.name, tuple(sorted(self.kwargs.items()))))


class BufferOpInstruction(PipeInstruction):
    def __init__(self, buffer_id, **kwargs):
        super().__init__(buffer_id=buffer_id, **kwargs)


class MultiStageOpInstruction(PipeInstruction):
    def __init__(self, stage_id, **kwargs):
        super().__init__(stage_id=stage_id, **kwargs)


class MultiStageBufferOpInstruction(BufferOpInstruction):
    def __init__(self, buffer_id, stage_id, **kwargs):
        super().__init__(buffer_id=buffer_id, stage_id=stage_id, **kwargs)


class CommunicationInstruction:
    """Marker base of the four p2p instructions."""


class LoadMicroBatch(BufferOpInstruction):
    pass


class ForwardPass(MultiStageBufferOpInstruction):
    pass


class BackwardPass(MultiStageBufferOpInstruction):
    pass


class SendActivation(MultiStageBufferOpInstruction, CommunicationInstruction):
    pass


class RecvActivation(MultiStageBufferOpInstruction, CommunicationInstruction):
    pass


class SendGrad(MultiStageBufferOpInstruction, CommunicationInstruction):
    pass


class RecvGrad(MultiStageBufferOpInstruction, CommunicationInstruction):
    pass


class SendWeights(MultiStageOpInstruction):
    pass


class RecvWeights(MultiStageOpInstruction):
    pass


class OptimizerStep(PipeInstruction):
    pass


class ReduceGrads(MultiStageOpInstruction):
    pass


class ReduceTiedGrads(PipeInstruction):
    pass


# --------------------------------------------------------------------------------- schedules
def _is_even(x):
    return x % 2 == 0


def _is_odd(x):
    return x % 2 != 0


def _step_to_micro_batch(stages, stage_id, step_id):
    """Map a 1F1B step to ``(micro_batch_id, is_forward)`` (reference schedule.py:6-46)."""
    if _is_even(step_id - stage_id):
        return (step_id - stage_id) // 2, True
    return (step_id + stage_id + 1) // 2 - stages, False


class PipeSchedule(ABC):
    """Iterable of per-step instruction lists for one stage."""

    def __init__(self, micro_batches, stages, stage_id):
        self.micro_batches = micro_batches
        self.stages = stages
        self.stage_id = stage_id
        self.prev_stage = stage_id - 1
        self.next_stage = stage_id + 1

    @abstractmethod
    def steps(self):
        ...

    def num_pipe_buffers(self):
        return self.micro_batches

    def _valid_micro_batch(self, micro_batch_id):
        return 0 <= micro_batch_id < self.micro_batches

    def _valid_stage(self, stage_id):
        return 0 <= stage_id < self.stages

    @property
    def stage(self):
        return self.stage_id

    @property
    def num_stages(self):
        return self.stages

    @property
    def num_micro_batches(self):
        return self.micro_batches

    @property
    def is_first_stage(self):
        return self.stage_id == 0

    @property
    def is_last_stage(self):
        return self.stage_id == self.stages - 1

    def _buffer_idx(self, micro_batch_id):
        assert self._valid_micro_batch(micro_batch_id)
        return micro_batch_id % self.num_pipe_buffers()

    def __iter__(self):
        self.it = None
        return self

    def __next__(self):
        if self.it is None:
            self.it = self.steps()
        return next(self.it)


class TrainSchedule(PipeSchedule):
    """1F1B training schedule of a stage; buffer id equals micro-batch id (M buffers)."""

    def __init__(self, micro_batches, stages, stage_id, **kwargs):
        super().__init__(micro_batches, stages, stage_id)

    @property
    def require_data_loader(self):
        return self.is_first_stage or self.is_last_stage

    def step_to_micro_batch(self, step_id):
        return _step_to_micro_batch(self.stages, self.stage_id, step_id)

    _step_to_micro_batch = step_to_micro_batch

    def valid_micro_batch(self, micro_batch_id):
        return self._valid_micro_batch(micro_batch_id)

    def steps(self):
        sid = self.stage_id
        upstream = self._valid_stage(self.prev_stage)
        downstream = self._valid_stage(self.next_stage)
        last = 2 * (self.micro_batches + self.stages - 1) - 1
        before = -1
        for t in range(last + 1):
            mb, forward = self.step_to_micro_batch(t)
            live = self._valid_micro_batch(mb)
            carried = self._valid_micro_batch(before)
            cmds = []
            if forward:
                if live and self.require_data_loader:
                    cmds.append(LoadMicroBatch(self._buffer_idx(mb)))
                if live and upstream:
                    cmds.append(RecvActivation(self._buffer_idx(mb), sid))
                if carried and upstream:
                    cmds.append(SendGrad(self._buffer_idx(before), sid))
                if live:
                    cmds.append(ForwardPass(self._buffer_idx(mb), sid))
            else:
                if carried and downstream:
                    cmds.append(SendActivation(self._buffer_idx(before), sid))
                if live and downstream:
                    cmds.append(RecvGrad(self._buffer_idx(mb), sid))
                if live:
                    cmds.append(BackwardPass(self._buffer_idx(mb), sid))
            if t == last:
                cmds += [ReduceGrads(sid), OptimizerStep()]
            before = mb
            yield cmds


class ResilientPipeSchedule(ABC):
    """Zips the stage's own schedule with its successor's and merges them step by step."""

    def __init__(self, sched, next_sched, failed_step=0, curr_step=0):
        self.sched = sched
        self.next_sched = next_sched
        self.failed_step = failed_step
        self.curr_step = curr_step
        self.cmd_buffer = []

    def steps(self):
        for i, (mine, theirs) in enumerate(zip(self.sched, self.next_sched)):
            yield self._merge_cmds(mine, theirs, i)

    def num_pipe_buffers(self):
        return self.sched.num_pipe_buffers()

    @abstractmethod
    def _merge_cmds(self, cmds, next_cmds, i):
        ...

    def __iter__(self):
        self.it = None
        return self

    def __next__(self):
        if self.it is None:
            self.it = self.steps()
        return next(self.it)


_RC_TYPES = (RecvActivation, LoadMicroBatch, ForwardPass)


class EagerRecoverySchedule(ResilientPipeSchedule):
    """Redundant computation: the successor's receive/load/forward commands are queued per
    step and the oldest queued step is issued in front of the next own step that waits on a
    gradient (``RecvGrad``), i.e. in the bubble where the stage would otherwise idle."""

    def _merge_cmds(self, cmds, next_cmds, i):
        merged = []
        waits_on_grad = any(type(c) is RecvGrad for c in cmds)
        if waits_on_grad and self.cmd_buffer:
            merged.extend(c for c in self.cmd_buffer.pop(0) if type(c) in _RC_TYPES)
        if any(type(c) in _RC_TYPES for c in next_cmds):
            self.cmd_buffer.append(next_cmds)
        merged.extend(cmds)
        return merged


class LazyRecoverySchedule(ResilientPipeSchedule):
    """No redundant computation; silent steps get a one-element ping (buffer id -1) so that a
    dead neighbour is noticed early."""

    def __init__(self, sched, next_sched, failed_step=0, curr_step=0):
        super().__init__(sched, next_sched, failed_step, curr_step)
        self.stage_id = sched.stage_id
        self.is_first_stage = sched.is_first_stage
        self.is_last_stage = sched.is_last_stage

    def _forward_step(self, stage_id, step_id):
        return _step_to_micro_batch(self.sched.stages, stage_id, step_id)[1]

    def _first_half(self, step_id):
        return step_id < self.sched.micro_batches + self.sched.stages - 1

    def _merge_cmds(self, cmds, next_cmds, i):
        sid = self.stage_id
        talks = any(isinstance(c, CommunicationInstruction) for c in cmds)
        fwd = self._forward_step(sid, i)
        ping_in, ping_out = RecvActivation(-1, sid), SendActivation(-1, sid)
        if self.is_first_stage:
            return [ping_in] + cmds if fwd else cmds
        if self.is_last_stage:
            if not talks and fwd and self._first_half(i):
                cmds = [ping_in] + cmds
            if self._forward_step(0, i):
                cmds = [ping_out] + cmds
            return cmds
        if not talks and self._first_half(i):
            cmds = [ping_in if fwd else ping_out] + cmds
        return cmds


class NextStageFailoverSchedule(ResilientPipeSchedule):
    """Stream of a stage that has absorbed its dead successor.

    Steps before ``curr_step`` replay the successor's commands only (its sends are dropped
    while ``i < failed_step``: the successor was still alive and had delivered them); from
    ``curr_step`` on both streams are interleaved and every own<->successor transfer becomes
    a local hand-off."""

    def _merge_cmds(self, cmds, next_cmds, i):
        if i < self.curr_step:
            if i < self.failed_step:
                return [c for c in next_cmds if type(c) not in (SendActivation, SendGrad)]
            return list(next_cmds)

        mine, theirs, merged = list(cmds), list(next_cmds), []
        while mine or theirs:
            a = type(mine[0]) if mine else None
            b = type(theirs[0]) if theirs else None
            if a is LoadMicroBatch:
                merged.append(mine.pop(0))
            elif a is RecvWeights:
                mine.pop(0)
            elif b is SendWeights:
                theirs.pop(0)
            elif b is LoadMicroBatch or b is SendActivation or b is RecvGrad:
                merged.append(theirs.pop(0))
            elif b is SendGrad:
                # successor -> own gradient: keep the own RecvGrad, served locally
                assert a is RecvGrad, f"Unable to merge cmds ({cmds}) and ({next_cmds})"
                theirs.pop(0)
                merged.append(mine.pop(0))
            elif b is RecvActivation:
                # own -> successor activation: keep the successor's RecvActivation
                assert a is SendActivation, f"Unable to merge cmds ({cmds}) and ({next_cmds})"
                mine.pop(0)
                merged.append(theirs.pop(0))
            elif a is BackwardPass:
                merged.append(mine.pop(0))
            elif b is BackwardPass:
                merged.append(theirs.pop(0))
            elif a is not None:
                merged.append(mine.pop(0))
            elif b in (ForwardPass, RecvWeights, ReduceGrads):
                merged.append(theirs.pop(0))
            elif b is OptimizerStep:
                theirs.pop(0)  # one optimizer step serves both stages
            else:
                raise Exception(f"Unable to merge cmds ({cmds}) and ({next_cmds})")
        return merged


class PrevStageFailoverSchedule(ResilientPipeSchedule):
    """Stream of the stage AFTER a dead one: re-send the gradients already delivered, then
    carry on with the own stream (``sched`` is ignored, ``next_sched`` is the own stream)."""

    def _merge_cmds(self, cmds, next_cmds, i):
        if i < self.curr_step:
            if i < self.failed_step:
                return [c for c in next_cmds if type(c) is SendGrad]
            return []
        keep = []
        for c in next_cmds:
            if type(c) is SendWeights:
                continue
            if type(c) is RecvActivation and c.buffer_id == -1:
                continue
            keep.append(c)
        return keep


class AllReduceFailoverSchedule(ResilientPipeSchedule):
    """Stream of a data-parallel peer of a dead rank: skip what ran before the failure."""

    def _merge_cmds(self, cmds, next_cmds, i):
        return [] if i < self.failed_step else cmds


class DataParallelSchedule(PipeSchedule):
    """Plain gradient accumulation on a single stage."""

    def steps(self):
        for step_id in range(self.micro_batches):
            cmds = [LoadMicroBatch(buffer_id=0), ForwardPass(buffer_id=0, stage_id=self.stage_id),
                    BackwardPass(buffer_id=0, stage_id=self.stage_id)]
            if step_id == self.micro_batches - 1:
                cmds += [ReduceGrads(self.stage_id), OptimizerStep()]
            yield cmds

    def num_pipe_buffers(self):
        return 1
