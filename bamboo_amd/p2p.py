"""In-process stand-in for the neighbours of a pipeline stage.

The reference moves activations and gradients between stages with ``dist.send`` /
``dist.recv`` (deepspeed/runtime/pipe/p2p_direct.py:11-17, called from engine.py:1894-2082).
On one GPU those transfers are replaced by a *seeded activation queue*: everything the
upstream stage would send and everything the downstream stage would send back is generated
once from seeds and kept resident in HBM, so a ``RecvActivation`` / ``RecvGrad`` is a buffer
lookup and a ``SendActivation`` / ``SendGrad`` is a hand-over to a sink.

Two kinds of downstream peer:
  * ``grad_mode="queue"``: the gradient of micro-batch ``k`` with respect to the output of stage
    ``s`` is a seeded N(0,1) tensor (a middle stage of a deeper pipeline);
  * ``grad_mode="mse"``: the peer is a loss head, ``loss_k = MSE(output_k, target_k)`` with seeded
    N(0,1) targets, gradient scaled by ``1 / micro_batches`` (the engine's loss scaling by the
    number of gradient-accumulation steps, deepspeed/runtime/engine.py:1430-1431).

Failure injection (the analogue of the reference's ``trigger_kill`` / p2p exceptions,
engine.py:407-416,1922-1930,2071-2079): ``preempt_successor(k)`` makes the transfers with the
successor of the own stage raise :class:`NextStageException` from micro-batch ``k`` on.
"""
import torch

from . import hip


class PrevStageException(Exception):
    ...


class NextStageException(Exception):
    ...


class AllReduceException(Exception):
    def __init__(self, src, *args):
        super().__init__(*args)
        self.src = src


class SeededActivationQueue:
    def __init__(self, shape, dtype, micro_batches, stage_ids, seed=1138, grad_mode="queue", device="cuda:0",
                 key_len_range=None, out_shapes=None):
        """shape: activation shape ``[micro_batch, seq, hidden]`` the stage receives, and the shape of every stage
        output unless ``out_shapes = {stage_id: shape}`` says otherwise (a down-sampling ResNet stage leaves fewer
        positions and more channels than it takes); stage_ids: stages whose *outputs* this queue must answer
        for (own stage and, for failover, the shadowed stage)."""
        self.out_shapes = {sid: tuple(s) for sid, s in (out_shapes or {}).items()}
        if grad_mode not in ("queue", "mse"):
            raise ValueError(grad_mode)
        self.shape, self.dtype, self.M = tuple(shape), dtype, micro_batches
        self.device, self.seed, self.grad_mode = torch.device(device), seed, grad_mode
        self.dead_from = None          # micro-batch id from which the successor is gone
        self.dead_stage = None
        self.sent = {}                 # (stage_id, k) -> tensor handed to the downstream peer
        self.sent_grads = {}
        self.loss = torch.zeros(1, dtype=torch.float32, device=self.device)
        self._mse_ws = torch.empty(hip.mse_workspace(), dtype=torch.float32, device=self.device)
        self.activations = [self._randn(("act", k)) for k in range(micro_batches)]
        self.key_lens = None
        if key_len_range is not None:
            lo, hi = key_len_range
            self.key_lens = []
            for k in range(micro_batches):
                g = torch.Generator().manual_seed(self._tag_seed(("len", k)))
                self.key_lens.append(torch.randint(lo, hi + 1, (shape[0],), generator=g, dtype=torch.int32).to(self.device))
        self.grads, self.targets = {}, {}
        for sid in stage_ids:
            out = self.out_shapes.get(sid, self.shape)
            if grad_mode == "queue":
                self.grads[sid] = [self._randn(("grad", sid, k), out) for k in range(micro_batches)]
            else:
                self.targets[sid] = [self._randn(("target", sid, k), out) for k in range(micro_batches)]
                self.grads[sid] = [torch.zeros(out, dtype=dtype, device=self.device) for _ in range(micro_batches)]

    _TAGS = {"act": 11, "grad": 23, "target": 37, "len": 41}

    def _tag_seed(self, tag):
        """Stable seed from (kind, ids...): independent of PYTHONHASHSEED."""
        h = self.seed
        for t in tag:
            h = (h * 1000003 + self._TAGS.get(t, t) + 7) % (2 ** 31 - 1)
        return h

    def _randn(self, tag, shape=None):
        g = torch.Generator().manual_seed(self._tag_seed(tag))
        return torch.randn(shape or self.shape, generator=g, dtype=torch.float32).to(self.dtype).to(self.device)

    # -------------------------------------------------------------- test hooks
    def set_grads(self, stage_id, tensors):
        """Replace the seeded output-gradients of ``stage_id`` (used to make the queue consistent
        with a real successor in failover tests)."""
        self.grads[stage_id] = [t.to(self.dtype).to(self.device).contiguous() for t in tensors]

    def preempt_successor(self, micro_batch, stage_id):
        """From ``micro_batch`` on, transfers between ``stage_id`` and its successor fail."""
        self.dead_from, self.dead_stage = micro_batch, stage_id

    def revive(self):
        self.dead_from = self.dead_stage = None

    def _check_alive(self, k, stage_id):
        if self.dead_from is not None and stage_id == self.dead_stage and k >= self.dead_from:
            raise NextStageException(f"successor of stage {stage_id} preempted at micro-batch {self.dead_from}")

    def start_batch(self):
        self.loss.zero_()
        self.sent.clear()
        self.sent_grads.clear()

    # -------------------------------------------------------------- p2p surface
    def recv_activation(self, k):
        return self.activations[k]

    def key_len(self, k):
        return None if self.key_lens is None else self.key_lens[k]

    def send_activation(self, k, tensor, stage_id, stream=None):
        self._check_alive(k, stage_id)
        self.sent[(stage_id, k)] = tensor
        if self.grad_mode == "mse":
            hip.mse_fwd_bwd(tensor, self.targets[stage_id][k], self.grads[stage_id][k], 1.0 / self.M, self.loss,
                            True, self._mse_ws, stream=stream)

    def recv_grad(self, k, stage_id):
        self._check_alive(k, stage_id)
        return self.grads[stage_id][k]

    def send_grad(self, k, tensor, stage_id):
        self.sent_grads[(stage_id, k)] = tensor

    def ping_next(self, stage_id):
        """One-element send from ``stage_id`` to its successor (``SendActivation(-1, stage_id)`` of the
        lazy schedule): fails like any other transfer with a successor that is gone."""
        if self.dead_from is not None and stage_id == self.dead_stage and self.dead_from <= 0:
            raise NextStageException(f"successor of stage {stage_id} does not answer")

    def ping_prev(self, stage_id):
        """One-element receive of ``stage_id`` from its predecessor (``RecvActivation(-1, stage_id)``).  This
        queue models the loss of a successor only; the activations it serves are always there."""
        return


# =============================================================================================
# A seeded queue that makes the stage wait as a real pipeline would: the bubbles of 1F1B
# =============================================================================================
import time  # noqa: E402


class PipelineClock:
    """Closed-loop model of the OTHER stages of an S-stage 1F1B pipeline around one real stage.

    Every other stage executes the forward / backward passes of its ``TrainSchedule`` stream in order; a
    forward takes ``t_fwd`` seconds, a backward ``t_bwd``; ``F(s, k)`` starts when stage ``s`` is free and
    ``F(s-1, k)`` has ended, ``B(s, k)`` when stage ``s`` is free and ``B(s+1, k)`` has ended (transfers
    take no time: the reference's p2p moves 17 MB over a link that does it in 0.1 ms).  The passes of the
    real stage enter with the times the GPU really finished them (:meth:`note_done`), so a real stage that
    falls behind delays its neighbours and, through them, what it receives later -- the loop is closed.

    What the real stage asks: when does ``RecvActivation(k)`` find its tensor (= end of ``F(s-1, k)``), when
    ``RecvGrad(k)`` (= end of ``B(s+1, k)``), and when does the whole pipeline finish the batch (= the last
    backward of stage 0)."""

    def __init__(self, stages, stage_id, micro_batches, t_fwd, t_bwd):
        from .schedule import BackwardPass, ForwardPass, TrainSchedule
        self.S, self.sid, self.M, self.t_fwd, self.t_bwd = stages, stage_id, micro_batches, float(t_fwd), float(t_bwd)
        self.order = {}     # stage -> [(kind, k)] in execution order
        self.before = {}    # (stage, kind, k) -> the pass the stage runs right before it
        for s in range(stages):
            seq = []
            for cmds in TrainSchedule(micro_batches=micro_batches, stages=stages, stage_id=s):
                for c in cmds:
                    if type(c) is ForwardPass:
                        seq.append(("F", c.buffer_id))
                    elif type(c) is BackwardPass:
                        seq.append(("B", c.buffer_id))
            self.order[s] = seq
            for i, (kind, k) in enumerate(seq):
                self.before[(s, kind, k)] = None if i == 0 else (s,) + seq[i - 1]
        self.start_batch(0.0)

    def start_batch(self, t0):
        """A batch whose first pass (stage 0's first forward) may start at ``t0`` (seconds on the clock's axis): 0 for
        a pipeline that starts empty, the previous batch's :meth:`pipeline_end` for batches run back to back."""
        self.t0 = t0
        self.end = {}        # (stage, kind, k) -> seconds on the clock's axis
        self.real = {}       # (kind, k) of the real stage -> callable returning seconds on that axis (blocks until known)

    def note_done(self, kind, k, when):
        """``when()``: the time on the clock's axis at which the real stage finished this pass (may block
        until the GPU has got there)."""
        self.real[(kind, k)] = when

    def end_of(self, s, kind, k):
        key = (s, kind, k)
        if key in self.end:
            return self.end[key]
        if s == self.sid:
            if (kind, k) not in self.real:
                raise RuntimeError(f"pipeline clock: {kind}({k}) of the real stage {s} is needed before it was issued")
            t = self.real[(kind, k)]()
        else:
            prev = self.before[key]
            t = self.t0 if prev is None else self.end_of(*prev)
            if kind == "F" and s > 0:
                t = max(t, self.end_of(s - 1, "F", k))
            if kind == "B" and s < self.S - 1:
                t = max(t, self.end_of(s + 1, "B", k))
            t += self.t_fwd if kind == "F" else self.t_bwd
        self.end[key] = t
        return t

    def activation_at(self, k):
        return self.end_of(self.sid - 1, "F", k) if self.sid > 0 else self.t0

    def grad_at(self, k):
        return self.end_of(self.sid + 1, "B", k) if self.sid < self.S - 1 else self.t0

    def pipeline_end(self):
        """When the last stage to finish the batch (stage 0, with its last backward) is done."""
        return max(self.end_of(s, *self.order[s][-1]) for s in range(self.S))


class PacedActivationQueue(SeededActivationQueue):
    """:class:`SeededActivationQueue` whose receives return when a real pipeline would deliver.

    ``RecvActivation(k)`` / ``RecvGrad(k)`` wait ON THE HOST (no kernel spins) until the moment a
    :class:`PipelineClock` gives for the tensor, then hand over the resident seeded tensor.  Because the
    engine issues a pass only after its receive has returned, the GPU really idles in the warm-up, wherever
    the stage is ahead of its neighbours, and in the cool-down: the bubbles of 1F1B exist, and what the
    engine has queued on another stream (redundant forwards) runs in them.  The stage's own passes are
    timed with events on their stream; their GPU completion times feed the clock."""

    def __init__(self, shape, dtype, micro_batches, stage_ids, stages, stage_id, t_fwd, t_bwd, **kw):
        super().__init__(shape, dtype, micro_batches, stage_ids, **kw)
        self.clock = PipelineClock(stages, stage_id, micro_batches, t_fwd, t_bwd)
        self.stage_id = stage_id
        self.waited = 0.0          # host seconds spent waiting for deliveries in this batch
        self.batch_seconds = None  # of the last finished batch: from its start to the pipeline's end
        self.batches = 0           # batches since the last reset()
        self._base = None
        self.rc_marks = None       # set to a list to collect (micro-batch, layer, "begin" | "end", seconds()) of redundant work

    def reset(self):
        """The next batch starts a new run: GPU drained, empty pipeline, time zero."""
        self._base = None

    def start_batch(self):
        """Batches run back to back: a batch starts on the pipeline's clock when the previous one has ended there
        (stage 0 is free for its first forward), whatever this stage's GPU still has queued -- redundant forwards left
        over from the previous batch run in the pipeline's fill time, as they would between real batches."""
        super().start_batch()
        if self._base is None:
            torch.cuda.synchronize(self.device)
            self._base = torch.cuda.Event(enable_timing=True)
            self._base.record(torch.cuda.current_stream(self.device))
            self._base.synchronize()
            self._t0 = time.perf_counter()
            self.clock.start_batch(0.0)
            self.batches = 0
        else:
            self.clock.start_batch(self._last_end)
        self.waited = 0.0

    def note_done(self, kind, k, stage_id, stream):
        """Called by the engine after it has issued forward / backward pass ``k`` of its own stage."""
        if stage_id != self.stage_id:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(stream)
        base = self._base

        def when():
            ev.synchronize()
            return base.elapsed_time(ev) * 1e-3
        self.clock.note_done(kind, k, when)

    def note_rc(self, k, layer, what, stream):
        """Called by the engine around every piece of a redundant forward it issues (layers ``begin`` .. ``end``
        of micro-batch ``k``); collected only while ``rc_marks`` is a list."""
        if self.rc_marks is None or self._base is None:
            return
        ev = torch.cuda.Event(enable_timing=True)
        ev.record(stream)
        base = self._base
        self.rc_marks.append((k, layer, what, lambda: base.elapsed_time(ev) * 1e-3))

    def _wait_until(self, t):
        target = self._t0 + t
        t_in = time.perf_counter()
        while True:
            left = target - time.perf_counter()
            if left <= 0:
                break
            time.sleep(min(left, 2e-4) if left > 3e-4 else 0)
        self.waited += time.perf_counter() - t_in

    def activation_arrived(self, k):
        """Non-consuming: has ``RecvActivation(k)`` nothing left to wait for?  (May itself wait for this stage's own
        earlier passes to finish on the GPU: what the neighbours send depends on them.)"""
        return time.perf_counter() >= self._t0 + self.clock.activation_at(k)

    def grad_arrived(self, k, stage_id):
        return stage_id != self.stage_id or time.perf_counter() >= self._t0 + self.clock.grad_at(k)

    def recv_activation(self, k):
        self._wait_until(self.clock.activation_at(k))
        return super().recv_activation(k)

    def recv_grad(self, k, stage_id):
        self._check_alive(k, stage_id)
        if stage_id == self.stage_id:
            self._wait_until(self.clock.grad_at(k))
        return super().recv_grad(k, stage_id)

    def end_batch(self, stage_ids):
        """The batch ends when the pipeline's last pass does (stage 0's last backward, which waits for every gradient
        this stage sends: the delays this stage caused are in it)."""
        self._last_end = self.clock.pipeline_end()
        self.batch_seconds = self._last_end - self.clock.t0
        self.batches += 1

    def finish(self):
        """Seconds from the start of the first batch after :meth:`reset` to the later of the pipeline's end of the
        last batch and the moment this stage's GPU work, redundant forwards included, has drained."""
        torch.cuda.synchronize(self.device)
        drained = time.perf_counter() - self._t0
        return max(self._last_end, drained)


# =============================================================================================
# Several stages in one process: a mailbox fabric between engines that run in threads
# =============================================================================================
import threading  # noqa: E402


class StageKilled(BaseException):
    """Raised inside the thread of a stage that the fabric preempts (the analogue of the spot
    instance disappearing): it unwinds ``train_batch`` of that engine and nothing else."""


class FabricTimeout(RuntimeError):
    ...


class LocalFabric:
    """Stage-to-stage transfers between engines of ONE process that share one GPU.

    Each engine runs ``train_batch`` in its own thread and blocks in ``recv_*`` until the
    neighbour has produced the tensor, as with ``dist.recv`` (p2p_direct.py:11-17).  All
    engines issue their kernels to the same HIP stream, so a tensor handed over here is ordered
    before its consumer's kernels without any further synchronisation.

    Messages are keyed by (batch, kind, producing stage, consuming stage, micro-batch), are not
    removed when read and are idempotent to re-send: after a stage is lost, its predecessor
    replays the lost stage's stream (``NextStageFailoverSchedule``) and finds everything the
    stage after it has sent, whether or not the dead stage had consumed it.

    Failure protocol of the reference (engine.py:1190-1303): both neighbours of the dead stage
    report the step at which they noticed (``fail-step-<rank>`` in the etcd store there,
    :meth:`FabricEndpoint.coordinate_fail_step` here) and continue from the smaller one.
    """

    def __init__(self, num_stages, shape, dtype, micro_batches, device="cuda:0", timeout=120.0):
        self.num_stages, self.shape, self.dtype, self.M = num_stages, tuple(shape), dtype, micro_batches
        self.device, self.timeout = torch.device(device), timeout
        self.cv = threading.Condition()
        self.box = {}
        self.dead = set()          # stages whose engine is gone and whose layers nobody has adopted yet
        self.kill_at = {}          # stage -> micro-batch at which its engine stops
        self.fail_steps = {}       # dead stage -> {reporting stage: step}
        self.finished = {}         # stage -> last batch it completed

    def endpoint(self, stage_id):
        return FabricEndpoint(self, stage_id)

    def kill(self, stage_id, at_micro_batch=0):
        """The engine of ``stage_id`` stops at its next transfer that concerns a micro-batch
        >= ``at_micro_batch`` (of the batch it is in)."""
        if stage_id in (0, self.num_stages - 1):
            raise ValueError("the first and the last stage have no two neighbours to recover them "
                             "(reference engine.py:1313-1315)")
        with self.cv:
            self.kill_at[stage_id] = at_micro_batch


class FabricEndpoint:
    """What one engine sees of the fabric: the ``activation_queue`` interface of
    :class:`SeededActivationQueue` for the stage(s) it hosts."""

    grad_mode = "queue"
    key_lens = None
    dead_from = dead_stage = None

    def __init__(self, fabric, stage_id):
        self.f, self.stage = fabric, stage_id
        self.shape, self.dtype, self.M, self.device = fabric.shape, fabric.dtype, fabric.M, fabric.device
        self.batch = -1
        self.acknowledged = set()  # dead stages whose loss this endpoint has already reported
        self.loss = torch.zeros(1, dtype=torch.float32, device=self.device)

    # ---------------------------------------------------------------- helpers
    def _check_kill(self, k):
        f = self.f
        with f.cv:
            at = f.kill_at.get(self.stage)
            if at is not None and k >= at:
                del f.kill_at[self.stage]
                f.dead.add(self.stage)
                f.cv.notify_all()
                raise StageKilled(f"stage {self.stage} preempted at micro-batch {k}")

    def _put(self, kind, src, dst, k, tensor, exc):
        f = self.f
        with f.cv:
            if dst in f.dead and dst not in self.acknowledged:
                raise exc(f"stage {dst} is gone ({kind} of micro-batch {k} from stage {src})")
            f.box[(self.batch, kind, src, dst, k)] = tensor
            f.cv.notify_all()

    def _get(self, kind, src, dst, k, exc):
        f = self.f
        key = (self.batch, kind, src, dst, k)
        waited = 0.0
        with f.cv:
            while key not in f.box:
                if src in f.dead and src not in self.acknowledged:
                    raise exc(f"stage {src} is gone ({kind} of micro-batch {k} for stage {dst})")
                if waited >= f.timeout:
                    raise FabricTimeout(f"stage {dst} waited {waited:.0f}s for {kind} {k} of stage {src}")
                f.cv.wait(0.5)
                waited += 0.5
            return f.box[key]

    # ---------------------------------------------------------------- queue interface
    def start_batch(self):
        self.batch += 1
        self.loss.zero_()
        f = self.f
        with f.cv:   # neighbours are never more than one batch apart
            for key in [key for key in f.box if isinstance(key[0], int) and key[0] < self.batch - 1]:
                del f.box[key]

    def end_batch(self, stage_ids):
        f = self.f
        with f.cv:
            for s in stage_ids:
                f.finished[s] = self.batch
            f.cv.notify_all()

    def key_len(self, k):
        return None

    def recv_activation(self, k):
        self._check_kill(k)
        return self._get("act", self.stage - 1, self.stage, k, PrevStageException)

    def send_activation(self, k, tensor, stage_id, stream=None):
        self._check_kill(k)
        self._put("act", stage_id, stage_id + 1, k, tensor, NextStageException)

    def recv_grad(self, k, stage_id):
        self._check_kill(k)
        return self._get("grad", stage_id + 1, stage_id, k, NextStageException)

    def send_grad(self, k, tensor, stage_id):
        self._check_kill(k)
        self._put("grad", stage_id, stage_id - 1, k, tensor, PrevStageException)

    def _ping(self, peer, exc):
        peer %= self.f.num_stages   # the pings of the first and the last stage close the ring (reference engine.py:_inc/_dec)
        with self.f.cv:
            if peer in self.f.dead and peer not in self.acknowledged:
                raise exc(f"stage {peer} does not answer")

    def ping_next(self, stage_id):
        """``SendActivation(-1, stage_id)``: a dead successor raises :class:`NextStageException`
        (reference engine.py:1903-1930)."""
        self._ping(stage_id + 1, NextStageException)

    def ping_prev(self, stage_id):
        """``RecvActivation(-1, stage_id)``: a dead predecessor raises :class:`PrevStageException`
        (reference engine.py:2012-2035)."""
        self._ping(stage_id - 1, PrevStageException)

    # ---------------------------------------------------------------- weights of a stage for its shadow
    def send_weights(self, stage_id, arenas):
        f = self.f
        with f.cv:
            f.box[("weights", stage_id)] = arenas
            f.cv.notify_all()

    def recv_weights(self, stage_id):
        with self.f.cv:
            return self.f.box.get(("weights", stage_id))

    # ---------------------------------------------------------------- whole layers (reconfiguration)
    def send_layer_tensors(self, dst_stage, layer_tensor, optim_tensor):
        f = self.f
        with f.cv:
            f.box[("layers", self.stage, dst_stage)] = (layer_tensor, optim_tensor)
            f.cv.notify_all()

    def recv_layer_tensors(self, src_stage):
        f = self.f
        key = ("layers", src_stage, self.stage)
        waited = 0.0
        with f.cv:
            while key not in f.box:
                if waited >= f.timeout:
                    raise FabricTimeout(f"stage {self.stage} waited {waited:.0f}s for layers of stage {src_stage}")
                f.cv.wait(0.5)
                waited += 0.5
            return f.box.pop(key)

    # ---------------------------------------------------------------- failure protocol
    def coordinate_fail_step(self, dead_stage, step):
        """Report the step at which this engine noticed that ``dead_stage`` is gone and return the
        smallest step reported by its neighbours (both of them unless the other one has already
        finished the batch without needing the dead stage any more)."""
        f = self.f
        other = dead_stage + 1 if self.stage < dead_stage else dead_stage - 1
        waited = 0.0
        with f.cv:
            self.acknowledged.add(dead_stage)
            reports = f.fail_steps.setdefault(dead_stage, {})
            reports[self.stage] = step
            f.cv.notify_all()
            while other not in reports and f.finished.get(other, -1) < self.batch:
                if waited >= f.timeout:
                    raise FabricTimeout(f"stage {self.stage}: no failure report from stage {other}")
                f.cv.wait(0.5)
                waited += 0.5
            return min(reports.values())

    def adopt(self, dead_stage):
        """The caller now runs the layers of ``dead_stage``: its transfers flow again."""
        f = self.f
        with f.cv:
            f.dead.discard(dead_stage)
            f.cv.notify_all()
