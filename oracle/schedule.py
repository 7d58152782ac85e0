"""Instruction streams of one pipeline stage, restated in closed form (TEST ORACLE).

An instruction is a tuple ``(name, buffer_id, stage_id)``; ``buffer_id`` /
``stage_id`` are ``None`` where the reference instruction does not carry them
(``OptimizerStep()``, ``ReduceGrads(stage_id)``, ``LoadMicroBatch(buffer_id)``).

Follows deepspeed/runtime/pipe/schedule.py of the reference:
  step_to_micro_batch   schedule.py:6-46
  train_schedule        schedule.py:225-310  (TrainSchedule.steps)
  eager_merge           schedule.py:504-524  (EagerRecoverySchedule._merge_cmds)
  next_stage_failover   schedule.py:343-430  (NextStageFailoverSchedule._merge_cmds)
  lazy_merge            schedule.py:469-501  (LazyRecoverySchedule._merge_cmds)
"""

RC_KINDS = ("RecvActivation", "LoadMicroBatch", "ForwardPass")


def step_to_micro_batch(stages, stage_id, step_id):
    """(micro_batch_id, is_forward) of a step.  A step is a forward step when its
    parity equals the stage's parity; forward id = (t - s)/2, backward id =
    (t + s + 1)/2 - S  (closed form of schedule.py:6-46)."""
    if (step_id - stage_id) % 2 == 0:
        return (step_id - stage_id) // 2, True
    return (step_id + stage_id + 1) // 2 - stages, False


def total_steps(micro_batches, stages):
    return 2 * (micro_batches + stages - 1)


def train_schedule(micro_batches, stages, stage_id):
    """List (one entry per step) of instruction lists of a 1F1B stage."""
    M, S, s = micro_batches, stages, stage_id
    valid = lambda k: 0 <= k < M
    has_prev, has_next = s > 0, s < S - 1
    loads = (s == 0) or (s == S - 1)
    out, prev = [], -1
    T = total_steps(M, S)
    for t in range(T):
        k, fwd = step_to_micro_batch(S, s, t)
        cmds = []
        if loads and fwd and valid(k):
            cmds.append(("LoadMicroBatch", k, None))
        if fwd:
            if valid(k) and has_prev:
                cmds.append(("RecvActivation", k, s))
            if valid(prev) and has_prev:
                cmds.append(("SendGrad", prev, s))
        else:
            if valid(prev) and has_next:
                cmds.append(("SendActivation", prev, s))
            if valid(k) and has_next:
                cmds.append(("RecvGrad", k, s))
        if valid(k):
            cmds.append(("ForwardPass" if fwd else "BackwardPass", k, s))
        if t == T - 1:
            cmds.append(("ReduceGrads", None, s))
            cmds.append(("OptimizerStep", None, None))
        prev = k
        out.append(cmds)
    return out


def eager_merge(own_steps, next_steps):
    """Eager redundant computation: the successor's Recv/Load/Forward commands of a
    step are queued, and the oldest queued step is emitted in front of the first
    later own step that holds a RecvGrad (schedule.py:504-524)."""
    fifo, out = [], []
    for own, nxt in zip(own_steps, next_steps):
        cmds = []
        if any(c[0] == "RecvGrad" for c in own) and fifo:
            cmds += [c for c in fifo.pop(0) if c[0] in RC_KINDS]
        if any(c[0] in RC_KINDS for c in nxt):
            fifo.append(nxt)
        out.append(cmds + list(own))
    return out


COMM_KINDS = ("SendActivation", "RecvActivation", "SendGrad", "RecvGrad")


def lazy_merge(own_steps, micro_batches, stages, stage_id):
    """Lazy recovery (schedule.py:483-501): no redundant work, the own stream plus one-element
    "pings" (buffer id -1) in front of some steps so that a dead neighbour is noticed while the
    stage would otherwise not talk to it.  Per step ``i`` of stage ``s`` (``half`` = the first
    ``M + S - 1`` steps, ``F(x)`` = step i is a forward step of stage x, ``quiet`` = the own step
    holds no send/recv):
      first stage:   listen (RecvActivation(-1)) on every F(s) step;
      last stage:    listen on quiet F(s) steps of the first half, and -- independently, placed in
                     front of it -- call (SendActivation(-1)) on every step that is F(0): the ring
                     last -> first;
      middle stages: on quiet steps of the first half, listen if F(s) else call."""
    M, S, s = micro_batches, stages, stage_id
    out = []
    for i, own in enumerate(own_steps):
        cmds = list(own)
        fwd = step_to_micro_batch(S, s, i)[1]
        quiet = not any(c[0] in COMM_KINDS for c in cmds)
        half = i < M + S - 1
        listen, call = ("RecvActivation", -1, s), ("SendActivation", -1, s)
        if s == 0:
            if fwd:
                cmds.insert(0, listen)
        elif s == S - 1:
            if quiet and fwd and half:
                cmds.insert(0, listen)
            if step_to_micro_batch(S, 0, i)[1]:
                cmds.insert(0, call)
        elif quiet and half:
            cmds.insert(0, listen if fwd else call)
        out.append(cmds)
    return out


def next_stage_failover(own_steps, next_steps, failed_step, curr_step):
    """Merged stream after the successor died (schedule.py:343-430).

    Steps before ``curr_step`` replay only the successor's commands (without its
    sends while ``< failed_step``); later steps interleave both streams by the
    eleven first-match rules of the reference."""
    out = []
    for i, (own, nxt) in enumerate(zip(own_steps, next_steps)):
        if i < curr_step:
            if i < failed_step:
                out.append([c for c in nxt if c[0] not in ("SendActivation", "SendGrad")])
            else:
                out.append(list(nxt))
            continue
        a, b, res = list(own), list(nxt), []
        while a or b:
            ha = a[0][0] if a else None
            hb = b[0][0] if b else None
            if ha == "LoadMicroBatch":
                res.append(a.pop(0))
            elif ha == "RecvWeights":
                a.pop(0)
            elif hb == "SendWeights":
                b.pop(0)
            elif hb == "LoadMicroBatch":
                res.append(b.pop(0))
            elif hb in ("SendActivation", "RecvGrad"):
                res.append(b.pop(0))
            elif hb == "SendGrad":
                assert ha == "RecvGrad", (own, nxt)
                b.pop(0)
                res.append(a.pop(0))
            elif hb == "RecvActivation":
                assert ha == "SendActivation", (own, nxt)
                a.pop(0)
                res.append(b.pop(0))
            elif ha == "BackwardPass":
                res.append(a.pop(0))
            elif hb == "BackwardPass":
                res.append(b.pop(0))
            elif ha is not None:
                res.append(a.pop(0))
            else:
                if hb in ("ForwardPass", "BackwardPass", "RecvWeights", "ReduceGrads"):
                    res.append(b.pop(0))
                elif hb == "OptimizerStep":
                    b.pop(0)
                else:
                    raise RuntimeError(f"cannot merge {own} and {nxt}")
        out.append(res)
    return out


def prev_stage_failover(own_steps, failed_step, curr_step):
    """Stream of the stage AFTER a lost one (schedule.py:433-454): steps it has already run are
    not run again, except that the gradients sent before ``failed_step`` are sent once more (the
    stage that replays the lost work has never received them); from ``curr_step`` on the own
    stream continues, without weight sends and without the lazy-mode pings."""
    out = []
    for i, own in enumerate(own_steps):
        if i < curr_step:
            out.append([c for c in own if c[0] == "SendGrad"] if i < failed_step else [])
        else:
            out.append([c for c in own if c[0] != "SendWeights" and not (c[0] == "RecvActivation" and c[1] == -1)])
    return out


def allreduce_failover(own_steps, failed_step):
    """Stream of a data-parallel peer of a lost rank (schedule.py:457-466): nothing before the
    failed step, the own stream from it on."""
    return [[] if i < failed_step else list(own) for i, own in enumerate(own_steps)]


def redundant_stage_ids(level, stage_id, stages):
    """Stages whose layers ``stage_id`` shadows (redundancy.py:7-19)."""
    return [(stage_id + i) % stages for i in range(1, level + 1)]


def redundant_user_stage_ids(level, stage_id, stages):
    """Stages that shadow ``stage_id`` (redundancy.py:22-31)."""
    return [i for i in range(stages) if stage_id in redundant_stage_ids(level, i, stages)]
