"""``PipelineEngine``: executes the instruction stream of one pipeline stage on one MI355X.

Surface of the reference engine (deepspeed/runtime/pipe/engine.py): constructor keywords
``redundancy_level, sync_save, eager_recovery`` (:104-105), ``train_batch(data_iter, debug,
mem_status, mem_log)`` (:1068-1423), attributes ``micro_batches, micro_batch_size, stage_id,
num_stages, stage_ids, r_stage_ids, pipe_buffers, global_steps``, the ``_exec_*`` handlers
and ``_INSTRUCTION_MAP`` (:1626-2147, :2324-2394), and the ``NextStageException`` failover
branch (:1190-1264).

What is different underneath:
  * layer arithmetic runs on the HIP kernels of ``libbamboo_hip.so`` with explicit backward
    passes; activations needed by a backward live in a per-stage HBM stash indexed by
    micro-batch (``buffer_id == micro_batch_id`` as in schedule.py:299-301);
  * stage-to-stage transfers are served by an in-process :class:`SeededActivationQueue`;
  * redundant forwards of the shadow stage can be issued to a second HIP stream so that the
    GPU overlaps them with the stage's own kernels (``rc_stream=True``); with either setting
    the shadow forward uses the same kernels, tiles and reduction order as a normal forward,
    so its output is bit-identical;
  * the Adam state of the shadow parameters is allocated up front, so promotion after a
    failure extends the optimizer without allocating (reference rebuilds FusedAdam,
    deepspeed/runtime/engine.py:306-333).
"""
import signal
import time
from collections import OrderedDict

import torch

from . import hip, schedule
from .config import BambooConfig
from .module import MirrorBuffer, PipelineError, PipelineModule, flat_mirror
from .optim import FusedAdam
from .p2p import AllReduceException, NextStageException, PrevStageException, SeededActivationQueue  # noqa: F401
from .utils import get_redundant_stage_ids, get_redundant_user_stage_ids

class PipelineEngine:
    def __init__(self, args=None, model=None, optimizer=None, model_parameters=None, training_data=None,
                 lr_scheduler=None, mpu=None, dist_init_required=None, collate_fn=None, config=None,
                 config_params=None, redundancy_level=0, sync_save=False, eager_recovery=False, prev_state={},
                 activation_queue=None, rc_stream=False, install_signal_handler=True, use_graphs=False,
                 rc_issue="reference", rc_backlog=None):
        if not isinstance(model, PipelineModule):
            raise PipelineError("model must base PipelineModule")
        hip.init()
        self.module = model
        cfg = config if config is not None else config_params
        if cfg is None and args is not None and getattr(args, "deepspeed_config", None):
            cfg = args.deepspeed_config
        self.config = cfg if isinstance(cfg, BambooConfig) else BambooConfig(cfg)
        if self.config.compute_dtype != model.dtype:
            raise PipelineError(f"config asks for {self.config.compute_dtype} but the module was built for {model.dtype}")
        # SIGTERM (the spot instance's preemption notice) makes the next train_batch exit with code 13
        # (reference engine.py:98-111, 1077-1079).  The flag lives on the engine; a process has one handler slot, so
        # with several engines in one process (one per thread) the last one built with the handler owns it.
        self.should_stop = False
        if install_signal_handler:
            signal.signal(signal.SIGTERM, self.sig_handler)

        self.device = model.device
        self.micro_batch_size = self.config.train_micro_batch_size_per_gpu
        self.micro_batches = self.config.gradient_accumulation_steps
        self.num_stages = model.num_stages
        self.stage_id = model.stage_id
        self.stage_ids = [self.stage_id]
        self.prev_stage = self.stage_id - 1
        self.next_stage = self.stage_id + 1
        self.dp_world_size = 1
        self.global_rank = 0
        self.global_steps = 0
        self.global_samples = 0
        self.training_data = training_data
        self.data_iterator = None
        self.lr_scheduler = lr_scheduler

        if redundancy_level > 1:
            raise NotImplementedError(f"R level {redundancy_level} > 1 is not supported now.")
        if eager_recovery and redundancy_level == 0:
            raise Exception("Must set redundancy level to enable eager recovery")
        self.redundancy_level = redundancy_level
        self.eager_recovery = eager_recovery
        self.sync_save = sync_save
        self.init_redundancy()

        self.queue = activation_queue
        if self.queue is None:
            raise PipelineError("activation_queue is required: it stands in for the neighbouring stages "
                                "(bamboo_amd.SeededActivationQueue)")
        if self.queue.shape[0] != self.micro_batch_size:
            raise PipelineError("activation queue micro-batch size differs from the config")
        self.batch, self.seq = self.queue.shape[0], self.queue.shape[1]

        # execution lanes: the stage's own work on the current stream, redundant forwards
        # optionally on a second stream of the same (default) priority
        self.main_stream = torch.cuda.current_stream(self.device)
        # Replay of the per-micro-batch launch sequences as HIP graphs: every forward or backward
        # of (stage, micro-batch) touches the same static buffers in every batch, so its ~100
        # launches are captured the second time they occur and launched as one graph afterwards.
        self.use_graphs = bool(use_graphs)
        if self.use_graphs and self._has_dropout(model.func_buckets):
            raise PipelineError("use_graphs with dropout: the dropout keys change with every batch and are kernel "
                                "arguments, a replayed graph would repeat the first batch's masks")
        if self.use_graphs and self.main_stream.cuda_stream == 0:
            raise PipelineError("use_graphs needs the engine built and run under a created stream "
                                "(torch.cuda.stream(...)): the default stream cannot be captured")
        self._graphs = {}
        self.rc_stream = torch.cuda.Stream(self.device) if (rc_stream and self.r_stage_ids and eager_recovery) else None
        # When a redundant forward is issued (results never depend on it, only timing):
        #   "reference": where EagerRecoverySchedule puts it, in front of the own step that waits for a gradient
        #                (schedule.py:504-524);
        #   "asap":      onto the second stream as soon as the own forward it depends on has been issued;
        #   "bubble":    into the pipeline's bubbles.  A redundant forward becomes *pending* once its input exists.
        #                Whenever the own stream is about to wait for a neighbour (a receive whose tensor is not
        #                there yet), pending forwards go to the second stream one layer at a time until the tensor
        #                arrives.  Only when more than `rc_backlog` are pending (the number the idle time behind the
        #                last own forward can absorb: cool-down, the wait for the stages in front to finish, the
        #                next batch's fill) is the oldest issued alongside own work; what is pending at the end of
        #                the batch is issued then.
        if rc_issue not in ("reference", "asap", "bubble"):
            raise PipelineError(f"rc_issue must be 'reference', 'asap' or 'bubble', got {rc_issue!r}")
        if rc_issue != "reference" and self.r_stage_ids and eager_recovery and self.rc_stream is None:
            raise PipelineError(f"rc_issue={rc_issue!r} needs rc_stream=True: on one stream an early redundant forward "
                                "would run in front of the own work instead of in its gaps")
        self.rc_issue = rc_issue
        # idle time behind the last own forward, in forward slots (a backward taken as two): S-1-s cool-down gaps,
        # s backward slots until stage 0 has finished, s forward slots until the next batch reaches this stage
        self.rc_backlog = rc_backlog if rc_backlog is not None else (self.num_stages - 1 - self.stage_id) + 3 * self.stage_id
        self._rc_pending = []      # micro-batches whose redundant forward is still to be issued, oldest first
        self._rc_partial = None    # [micro-batch, next layer, its input] of a forward issued layer by layer
        self._rc_forced = False
        self._own_tail = None      # event behind the last pass issued to the own stream
        built = list(self.stage_ids) + (list(self.r_stage_ids) if self.eager_recovery else [])
        self.ctx = model.prepare_context(built, self.batch, self.seq, stream=self.main_stream)
        self.rc_ctx = self.ctx
        if self.rc_stream is not None:
            # the shadowed stage takes what the own stage leaves (a down-sampling stage changes the positions)
            self.rc_ctx = model.prepare_context(self.r_stage_ids, self.batch, model.stage_seq[self.r_stage_ids[0]][0],
                                                stream=self.rc_stream, forward_only=True)
        self.stash_bytes = 0
        for sid in built:
            self.stash_bytes += model.allocate_stash(sid, self.ctx, self.micro_batches)
        self._fwd_done = [torch.cuda.Event() for _ in range(self.micro_batches)]
        self._deferred = {}   # (stage, slot) -> the slot's last forward left backward-only outputs out

        if model.stage_io_shapes(self.stage_id, self.batch)[0] != (self.batch * self.seq, self.queue.shape[2]):
            raise PipelineError(f"the activation queue delivers {tuple(self.queue.shape)}, the stage's first layer takes "
                                f"{model.stage_io_shapes(self.stage_id, self.batch)[0]} (rows, features)")
        self._input_grad_store = {
            sid: [torch.empty(model.stage_io_shapes(sid, self.batch)[0], dtype=model.dtype, device=self.device)
                  for _ in range(self.micro_batches)]
            for sid in built}
        self._loss_grad = None     # gradient of the loss head: allocated with the first last-stage output it sees
        self.total_loss = torch.zeros(1, dtype=torch.float32, device=self.device)

        self.optimizer = optimizer if optimizer is not None else FusedAdam(
            lr=self.config.lr, betas=self.config.betas, eps=self.config.eps, weight_decay=self.config.weight_decay,
            adam_w_mode=self.config.adam_w_mode, bias_correction=self.config.bias_correction)
        self.optimizer.add_stage(self.stage_id, model.stage_params[self.stage_id])

        self.init_pipe_buffers()
        self._failover = None          # (failed_step, curr_step) once the successor is absorbed
        self._prev_failover = None     # (failed_step, curr_step) once the predecessor has been replaced
        self.last_failover = None      # timing record of the most recent promotion
        self._install_sched_generator()
        self.tput_t0 = None
        self.timers = {}

    def _has_dropout(self, stage_ids):
        return any(getattr(layer, "dropout", 0) > 0 for sid in stage_ids for layer in self.module.func_buckets.get(sid, []))

    def sig_handler(self, signum, frame):
        print("[Engine] Signal handler called with signal", signum)
        self.should_stop = True

    def set_gemm_hook(self, hook):
        """Observer of every GEMM launch of THIS engine's lanes (``hook(desc, launch, stream)``, see ``hip.gemm``), or
        None.  While one is set the engine launches eagerly (a captured graph would replay the launches past it)."""
        self.ctx.gemm_hook = hook
        self.rc_ctx.gemm_hook = hook

    # ------------------------------------------------------------------ redundancy
    def _inc(self, stage_id):
        return (stage_id + 1) % self.num_stages

    def _dec(self, stage_id):
        return (stage_id - 1 + self.num_stages) % self.num_stages

    def init_redundancy(self):
        """Decide which stage is shadowed and materialise its layers (eager mode) or zero CPU
        mirrors of its parameters and Adam state (lazy mode); reference engine.py:317-350."""
        self.r_stage_ids = get_redundant_stage_ids(self.redundancy_level, self.stage_id, self.num_stages)
        self.r_user_stage_ids = get_redundant_user_stage_ids(self.redundancy_level, self.stage_id, self.num_stages)
        self.param_buffers, self.state_buffers = {}, {}
        for sid in self.r_stage_ids:
            self.param_buffers[sid], self.state_buffers[sid] = MirrorBuffer(), MirrorBuffer()
            if self.eager_recovery:
                self.module.build_layers(sid)
                for name, p in self.module.get_named_param(sid):
                    self.param_buffers[sid][name] = p
                sp = self.module.stage_params[sid]
                for i, name in enumerate(sp.index):
                    self.state_buffers[sid][f"{i}.exp_avg"] = sp.view(sp.exp_avg, name)
                    self.state_buffers[sid][f"{i}.exp_avg_sq"] = sp.view(sp.exp_avg_sq, name)
            else:
                names = self.module.allocate_param(sid, self.param_buffers[sid], "cpu")
                # both moments of a parameter as views of two flat host tensors in the arena's order
                total = self.param_buffers[sid].flat.numel()
                flats = {"exp_avg": flat_mirror(total), "exp_avg_sq": flat_mirror(total)}
                off = 0
                for i, name in enumerate(names):
                    z = self.param_buffers[sid][name]
                    for kind, flat in flats.items():
                        self.state_buffers[sid][f"{i}.{kind}"] = flat[off: off + z.numel()].view(z.shape)
                    off += z.numel()
                self.state_buffers[sid].flat = flats

    def init_pipe_buffers(self):
        """Per-micro-batch buffer lists keyed like the reference's (engine.py:352-387)."""
        self.num_pipe_buffers = 0
        self.pipe_buffers = {"data": [], "label": [], f"input_{self.stage_id}": [], f"output_{self.stage_id}": []}
        if self.stage_id != 0:
            self.pipe_buffers[f"input_grad_{self.stage_id}"] = []
        if self.eager_recovery:
            for sid in self.r_stage_ids:
                self.pipe_buffers[f"input_{sid}"] = []
                self.pipe_buffers[f"output_{sid}"] = []
                self.pipe_buffers[f"input_grad_{sid}"] = []
        self.grad_layer = {}

    def _reserve_pipe_buffers(self, num_buffers):
        for key in self.pipe_buffers:
            cur = self.pipe_buffers[key]
            cur.extend([None] * (num_buffers - len(cur)))
        self.num_pipe_buffers = max(self.num_pipe_buffers, num_buffers)

    def _clean_pipe_buffers(self):
        for key in self.pipe_buffers:
            self.pipe_buffers[key] = [None] * len(self.pipe_buffers[key])

    # ------------------------------------------------------------------ schedules
    def _train_sched(self, stage_id):
        return schedule.TrainSchedule(micro_batches=self.micro_batches, stages=self.num_stages, stage_id=stage_id)

    def _install_sched_generator(self):
        if self._failover is not None:
            own, absorbed = self.stage_ids[0], self.stage_ids[1]
            fs, cs = self._failover
            base = lambda: schedule.NextStageFailoverSchedule(
                self._train_sched(own), self._train_sched(absorbed), failed_step=fs, curr_step=cs)
        elif self.r_stage_ids:
            cls = schedule.EagerRecoverySchedule if self.eager_recovery else schedule.LazyRecoverySchedule
            nxt = self.r_stage_ids[0]
            base = lambda: cls(self._train_sched(self.stage_id), self._train_sched(nxt))
        else:
            base = lambda: self._train_sched(self.stage_id)
        if self._prev_failover is not None:
            # the stage in front of this one was lost and is now run by ITS predecessor
            # (reference engine.py:1266-1303): re-send what the lost stage had been given, then carry on
            fs, cs = self._prev_failover
            self._generate_sched = lambda: schedule.PrevStageFailoverSchedule(
                self._train_sched(self.prev_stage), base(), failed_step=fs, curr_step=cs)
        else:
            self._generate_sched = base

    # ------------------------------------------------------------------ properties
    def is_first_stage(self):
        return self.stage_id == 0

    def is_last_stage(self):
        return self.stage_id == self.num_stages - 1

    def train_batch_size(self):
        return self.config.train_batch_size

    def train_micro_batch_size_per_gpu(self):
        return self.micro_batch_size

    def gradient_accumulation_steps(self):
        return self.micro_batches

    def steps_per_print(self):
        return self.config.steps_per_print

    def wall_clock_breakdown(self):
        return self.config.wall_clock_breakdown

    def set_dataiterator(self, iterator):
        self.data_iterator = iterator

    def forward(self, *args, **kwargs):
        raise PipelineError("Only train_batch() is accessible in pipeline mode.")

    def backward(self, *args, **kwargs):
        raise PipelineError("Only train_batch() is accessible in pipeline mode.")

    def step(self, *args, **kwargs):
        raise PipelineError("Only train_batch() is accessible in pipeline mode.")

    def log(self, msg):
        print(f"[ {self.global_rank:02d}|{self.global_steps:02d} ] {msg}", flush=True)

    def mem_status(self, msg, print_rank=-1, reset_max=False):
        alloc = torch.cuda.memory_allocated(self.device) / 2 ** 30
        peak = torch.cuda.max_memory_allocated(self.device) / 2 ** 30
        self.log(f"MEMSTATS {msg} current alloc={alloc:.2f}GB (peak {peak:.2f}GB) stash={self.stash_bytes / 2 ** 30:.2f}GB")
        if reset_max:
            torch.cuda.reset_peak_memory_stats(self.device)

    # ------------------------------------------------------------------ train_batch
    def train_batch(self, data_iter=None, debug=False, mem_status=False, mem_log=False):
        """Run one batch (``micro_batches`` micro-batches) through the stage's schedule, including
        the redundant forwards and, if the successor is lost, the failover; returns the mean
        micro-batch loss where this process sees one (loss-head peer or last stage), else 0."""
        if self.should_stop:
            raise SystemExit(13)
        if data_iter is not None:
            self.set_dataiterator(data_iter)
        elif self.data_iterator is None and self.training_data is not None:
            self.data_iterator = iter(self.training_data)
        self._reserve_pipe_buffers(self.micro_batches)
        self.queue.start_batch()
        self.total_loss.zero_()
        self._loss_done = set()
        self._rc_forced = False
        self._debug = debug
        t0 = time.perf_counter()

        self.check_preemptions()
        status = self._exec_schedule(self._generate_sched())
        if status is not None:
            step_i, exc = status
            if isinstance(exc, NextStageException) and self.r_stage_ids:
                self._handle_next_stage_failure(step_i)
                status = self._exec_schedule(self._generate_sched())
                if status is not None:
                    raise status[1]
                # later batches run the merged stream from its first step
                self._failover = (0, 0)
                self._install_sched_generator()
            elif isinstance(exc, PrevStageException) and hasattr(self.queue, "coordinate_fail_step"):
                self._handle_prev_stage_failure(step_i)
                status = self._exec_schedule(self._generate_sched())
                if status is not None:
                    raise status[1]
                self._prev_failover = (0, 0)
                self._install_sched_generator()
            else:
                raise exc
        if self.rc_issue == "bubble" and self.r_stage_ids:
            self._rc_flush()     # runs while the stages in front finish the batch and the next one fills the pipeline
        if hasattr(self.queue, "end_batch"):
            self.queue.end_batch(self.stage_ids)
        if self.rc_stream is not None:
            self.main_stream.wait_stream(self.rc_stream)

        if self.queue.grad_mode == "mse":
            loss = self.queue.loss / self.micro_batches
        else:
            loss = self.total_loss / self.micro_batches
        self.agg_train_loss = loss

        if self.global_steps % self.steps_per_print() == 0 and (debug or self.wall_clock_breakdown()):
            torch.cuda.synchronize(self.device)
            elapsed = time.perf_counter() - t0
            self.log(f"steps: {self.global_steps} loss: {float(loss):0.4f} iter time (s): {elapsed:0.3f} "
                     f"samples/sec: {self.train_batch_size() / elapsed:0.3f}")
        if mem_status or mem_log:
            self.mem_status("AFTER BATCH")
        self._clean_pipe_buffers()
        return loss

    def check_preemptions(self):
        """Announced preemption (reference engine.py:731-809): if the successor is already known to
        be gone before the batch starts, absorb it now and run the merged stream from step 0."""
        q = self.queue
        if (self._failover is None and self.r_stage_ids and q.dead_from is not None and q.dead_from <= 0
                and q.dead_stage == self.stage_id):
            self._promote(self.r_stage_ids[0], failed_step=0, curr_step=0)

    def _handle_next_stage_failure(self, step_i):
        torch.cuda.synchronize(self.device)   # the pause starts when the work issued before the failure has drained
        t0 = time.perf_counter()
        nxt = self.r_stage_ids[0]
        if hasattr(self.queue, "coordinate_fail_step"):
            # both neighbours of the lost stage agree on the earlier of the two steps at which they
            # noticed (reference engine.py:1207-1222)
            failed_step = self.queue.coordinate_fail_step(nxt, step_i)
        else:
            # the seeded queue has seen nothing of the dead successor's traffic with the stage after
            # it, so the replay keeps the successor's sends (the second replay case of the
            # reference, schedule.py:349-353)
            failed_step = 0
        # micro-batches whose own forward has run but whose redundant forward has not (held back for a bubble, issued
        # in part, or simply not due yet where the schedule places it): the replay computes these first
        own_out, rc_out = self.pipe_buffers[f"output_{self.stage_id}"], self.pipe_buffers.get(f"output_{nxt}", [])
        partial = self._rc_partial[0] if self._rc_partial is not None else None
        missing = sum(1 for k, o in enumerate(own_out)
                      if o is not None and (k >= len(rc_out) or rc_out[k] is None or k == partial))
        self._promote(nxt, failed_step=failed_step, curr_step=step_i)
        if hasattr(self.queue, "adopt"):
            self.queue.adopt(nxt)
        self.last_failover = {"step": step_i, "failed_step": failed_step, "t_detect": t0,
                              "promote_s": time.perf_counter() - t0, "rc_missing": missing}
        self._replay_until = step_i

    def _handle_prev_stage_failure(self, step_i):
        """The stage in front of this one is gone (reference engine.py:1266-1303): agree on the
        failed step with the stage that takes its place and switch to the stream that re-sends the
        gradients of the steps before it."""
        failed_step = self.queue.coordinate_fail_step(self.prev_stage, step_i)
        self._prev_failover = (failed_step, step_i)
        self._install_sched_generator()
        self.last_failover = {"step": step_i, "failed_step": failed_step, "role": "successor of the lost stage"}

    def _promote(self, absorbed, failed_step, curr_step):
        """Turn the shadow layers of ``absorbed`` into active layers of this process
        (reference engine.py:1190-1264)."""
        if not self.eager_recovery:
            # lazy mode keeps CPU mirrors only: materialise the layers from them now
            self.module.build_layers(absorbed, self.param_buffers[absorbed])
            if self.use_graphs and self._has_dropout([absorbed]):
                # the layers that arrive only now carry dropout (the constructor's check saw the own stage alone):
                # from here on every kernel is launched with this batch's keys, nothing is replayed
                self.use_graphs = False
                self._graphs.clear()
            sp = self.module.stage_params[absorbed]
            flats = getattr(self.state_buffers[absorbed], "flat", None)
            if flats is not None and flats["exp_avg"].numel() == sp.numel:
                sp.exp_avg.copy_(flats["exp_avg"])          # one transfer per moment arena
                sp.exp_avg_sq.copy_(flats["exp_avg_sq"])
            else:
                for i, name in enumerate(sp.index):
                    sp.view(sp.exp_avg, name).copy_(self.state_buffers[absorbed][f"{i}.exp_avg"])
                    sp.view(sp.exp_avg_sq, name).copy_(self.state_buffers[absorbed][f"{i}.exp_avg_sq"])
            hook = self.ctx.gemm_hook
            self.ctx = self.module.prepare_context(self.stage_ids + [absorbed], self.batch, self.seq, stream=self.main_stream)
            self.ctx.gemm_hook = hook
            self.stash_bytes += self.module.allocate_stash(absorbed, self.ctx, self.micro_batches)
            act_shape = self.module.stage_io_shapes(absorbed, self.batch)[0]
            self._input_grad_store[absorbed] = [torch.empty(act_shape, dtype=self.module.dtype, device=self.device)
                                                for _ in range(self.micro_batches)]
            for key in (f"input_{absorbed}", f"output_{absorbed}", f"input_grad_{absorbed}"):
                self.pipe_buffers[key] = [None] * self.micro_batches
        if self.rc_stream is not None:
            self.main_stream.wait_stream(self.rc_stream)
        # redundant forwards not issued, or issued in part: the replay runs them as ordinary forwards
        self._rc_pending, self._rc_partial = [], None
        self.rc_ctx = self.ctx
        self.optimizer.add_stage(absorbed, self.module.stage_params[absorbed])
        self.stage_ids.append(absorbed)
        self.r_stage_ids = []
        self.next_stage = self._inc(absorbed)
        self._failover = (failed_step, curr_step)
        self._install_sched_generator()

    # ------------------------------------------------------------------ graph replay
    def _graphed(self, key, stream, issue):
        """Run ``issue()`` (which only launches kernels of this library on ``stream`` and returns a
        value that does not change between batches): eagerly the first time ``key`` occurs, captured
        and launched the second time, replayed from then on."""
        if not self.use_graphs or self.ctx.gemm_hook is not None:
            return issue()
        state = self._graphs.get(key)
        if state is None:
            self._graphs[key] = "seen"
            return issue()
        if state == "seen":
            with hip.Graph.capture(stream) as graph:
                out = issue()
            self._graphs[key] = (graph, out)
        graph, out = self._graphs[key]
        graph.launch(stream)
        return out

    # ------------------------------------------------------------------ instruction handlers
    def _exec_load_micro_batch(self, buffer_id):
        if self.pipe_buffers["label"][buffer_id] is not None or self.pipe_buffers["data"][buffer_id] is not None:
            return
        if self.data_iterator is None:
            raise PipelineError("LoadMicroBatch needs training_data or a data_iter")
        batch = next(self.data_iterator)
        hosted = self.stage_ids + self.r_stage_ids
        if 0 in hosted:
            x = batch[0].to(self.device).to(self.module.dtype)
            self.pipe_buffers["data"][buffer_id] = x.reshape(-1, x.shape[-1]).contiguous()
        if self.num_stages - 1 in hosted:
            y = batch[1].to(self.device).to(self.module.dtype)
            self.pipe_buffers["label"][buffer_id] = y.reshape(-1, y.shape[-1]).contiguous()

    def _exec_recv_activations(self, buffer_id, stage_id):
        if buffer_id == -1:
            # one-element receive from the predecessor (reference engine.py:2012-2035): a dead
            # predecessor surfaces as PrevStageException
            self.queue.ping_prev(stage_id)
            return
        key = f"input_{stage_id}"
        if self.pipe_buffers[key][buffer_id] is not None:
            return
        producer = stage_id - 1
        if producer in self.stage_ids:
            # local hand-off: the producer's output buffer stays valid until the end of the batch
            self.pipe_buffers[key][buffer_id] = self.pipe_buffers[f"output_{producer}"][buffer_id]
        else:
            if hasattr(self.queue, "activation_arrived"):
                self._fill_bubble(lambda: self.queue.activation_arrived(buffer_id))
            x = self.queue.recv_activation(buffer_id)
            self.pipe_buffers[key][buffer_id] = x.view(-1, x.shape[-1])

    def _exec_send_activations(self, buffer_id, stage_id):
        if buffer_id == -1:
            # one-element send to the successor (reference engine.py:1903-1930): a dead successor
            # surfaces as NextStageException
            self.queue.ping_next(stage_id)
            return
        if stage_id + 1 in self.stage_ids:
            return
        out = self.pipe_buffers[f"output_{stage_id}"][buffer_id]
        self.queue.send_activation(buffer_id, out, stage_id, stream=self.main_stream)

    def _exec_recv_grads(self, buffer_id, stage_id):
        if stage_id + 1 in self.stage_ids:
            self.grad_layer[stage_id] = self.pipe_buffers[f"input_grad_{stage_id + 1}"][buffer_id]
        else:
            if hasattr(self.queue, "grad_arrived"):
                self._fill_bubble(lambda: self.queue.grad_arrived(buffer_id, stage_id))
            g = self.queue.recv_grad(buffer_id, stage_id)
            self.grad_layer[stage_id] = g.view(-1, g.shape[-1])

    def _exec_send_grads(self, buffer_id, stage_id):
        if stage_id - 1 in self.stage_ids:
            return
        self.queue.send_grad(buffer_id, self.pipe_buffers[f"input_grad_{stage_id}"][buffer_id], stage_id)

    def _exec_forward_pass(self, buffer_id, stage_id):
        out_key = f"output_{stage_id}"
        last_with_loss = stage_id == self.num_stages - 1 and self.module.loss_fn is not None
        if self.pipe_buffers[out_key][buffer_id] is not None:
            # The reference keeps no output of the last stage (engine.py:1646), so a replayed forward of
            # an absorbed last stage computes the loss again.  Here the redundant forward's output is
            # kept for the backward pass from the stash, and only the loss head still has to run on it.
            if (last_with_loss and stage_id in self.stage_ids and self._deferred.get((stage_id, buffer_id))
                    and (stage_id, buffer_id) not in self._loss_done):
                self._loss_head(buffer_id, stage_id, self.pipe_buffers[out_key][buffer_id])
            return
        inputs = self.pipe_buffers["data" if stage_id == 0 else f"input_{stage_id}"][buffer_id]
        redundant = stage_id in self.r_stage_ids
        if redundant and self.rc_issue == "bubble" and not self._rc_forced:
            return      # issued from the bubbles, the backlog limit or the end of the batch instead
        ctx = self.rc_ctx if redundant else self.ctx
        ctx.key_len = self.queue.key_len(buffer_id)
        ctx.redundant = redundant
        # what names this micro-batch's dropout masks: the same for the redundant forward, the normal forward of
        # the same layers, a replay and the backward pass (the reference reseeds per layer and micro-batch for
        # the same purpose, deepspeed/runtime/pipe/module.py:538-545)
        ctx.dropout_base = (self.module.base_seed, self.global_steps, buffer_id)
        if redundant and self.rc_stream is not None:
            self.rc_stream.wait_event(self._fwd_done[buffer_id])
        kl = ctx.key_len
        key = ("F", stage_id, buffer_id, id(ctx), inputs.data_ptr(), None if kl is None else kl.data_ptr())
        # a redundant forward's stash is read by a backward pass only after a failover: it leaves out
        # what that backward pass can produce itself
        self._deferred[(stage_id, buffer_id)] = redundant
        note_rc = getattr(self.queue, "note_rc", None) if redundant else None
        if note_rc is not None:      # a queue that keeps a timeline of the redundant work (measurement only)
            note_rc(buffer_id, 0, "begin", ctx.stream)
        out = self._graphed(key, ctx.stream, lambda: self.module.forward(inputs, stage_id, slot=buffer_id, ctx=ctx,
                                                                         defer=redundant))
        if note_rc is not None:
            note_rc(buffer_id, len(self.module.func_buckets[stage_id]), "end", ctx.stream)
        self.pipe_buffers[out_key][buffer_id] = out
        if not redundant and self.rc_stream is not None:
            self._fwd_done[buffer_id].record(self.main_stream)
        if not redundant and hasattr(self.queue, "note_done"):
            self.queue.note_done("F", buffer_id, stage_id, self.main_stream)
        if not redundant and self.rc_issue == "bubble":
            self._mark_own_tail()
        if (not redundant and self.rc_stream is not None and stage_id == self.stage_id and self.r_stage_ids
                and self.eager_recovery):
            if self.rc_issue == "asap":
                self._rc_issue_whole(buffer_id)
            elif self.rc_issue == "bubble":
                self._rc_pending.append(buffer_id)
                while len(self._rc_pending) > self.rc_backlog:
                    self._rc_issue_oldest()
        if last_with_loss and not redundant:
            self._loss_head(buffer_id, stage_id, out)

    # ------------------------------------------------------------------ redundant forwards outside the stream's order
    def _rc_issue_whole(self, k):
        """The redundant forward of micro-batch ``k`` now (second stream, behind the own forward it reads)."""
        nxt = self.r_stage_ids[0]
        if nxt == self.num_stages - 1 and self.data_iterator is not None:
            self._exec_load_micro_batch(k)
        self._rc_forced = True
        try:
            self._exec_recv_activations(k, nxt)
            self._exec_forward_pass(k, nxt)
        finally:
            self._rc_forced = False

    def _rc_issue_oldest(self):
        """Issue what is left of the oldest pending redundant forward in one go."""
        k = self._rc_pending[0]
        if self._rc_partial is not None and self._rc_partial[0] == k:
            while self._rc_issue_layer() is not None and self._rc_partial is not None:
                pass
            return
        self._rc_pending.pop(0)
        self._rc_issue_whole(k)

    def _rc_issue_layer(self):
        """Issue ONE layer of the oldest pending redundant forward on the second stream; returns an event that
        completes with it (None when nothing is pending).  Same kernels on the same operands as the whole forward:
        the result does not depend on how the forward was cut."""
        if not self._rc_pending:
            return None
        k, nxt = self._rc_pending[0], self.r_stage_ids[0]
        n_layers = len(self.module.func_buckets[nxt])
        if self.module.activation_checkpoint_interval > 0:
            self._rc_pending.pop(0)      # checkpointed stashes are filled by whole forwards only
            self._rc_issue_whole(k)
        else:
            ctx = self.rc_ctx
            if self._rc_partial is None or self._rc_partial[0] != k:
                if nxt == self.num_stages - 1 and self.data_iterator is not None:
                    self._exec_load_micro_batch(k)
                self._exec_recv_activations(k, nxt)
                self.rc_stream.wait_event(self._fwd_done[k])
                self._rc_partial = [k, 0, self.pipe_buffers[f"input_{nxt}"][k]]
                self._deferred[(nxt, k)] = True
            _, i, x = self._rc_partial
            ctx.key_len = self.queue.key_len(k)
            ctx.redundant = True
            ctx.dropout_base = (self.module.base_seed, self.global_steps, k)
            note_rc = getattr(self.queue, "note_rc", None)
            if note_rc is not None:
                note_rc(k, i, "begin", self.rc_stream)
            out = self.module.forward(x, nxt, slot=k, ctx=ctx, defer=True, layers=(i, i + 1))
            if note_rc is not None:
                note_rc(k, i + 1, "end", self.rc_stream)
            if i + 1 == n_layers:
                self.pipe_buffers[f"output_{nxt}"][k] = out
                self._rc_pending.pop(0)
                self._rc_partial = None
            else:
                self._rc_partial = [k, i + 1, out]
        ev = torch.cuda.Event()
        ev.record(self.rc_stream)
        return ev

    def _fill_bubble(self, arrived):
        """The own stream is about to wait for a neighbour: pending redundant forwards go out, one layer at a time,
        until ``arrived()`` says the awaited tensor is there (the layer in flight then overlaps the own pass that
        follows, for a fraction of a millisecond)."""
        if self.rc_issue != "bubble" or self.rc_stream is None or not self.r_stage_ids:
            return
        while self._rc_pending and not arrived():
            if self._own_tail is not None and not self._own_tail.query():
                time.sleep(0)      # the host is ahead of the GPU: the own stream still has work, this is no bubble yet
                continue
            ev = self._rc_issue_layer()
            while ev is not None and not ev.query():
                if arrived():
                    return
                time.sleep(0)

    def _mark_own_tail(self):
        self._own_tail = torch.cuda.Event()
        self._own_tail.record(self.main_stream)

    def _rc_flush(self):
        """End of the batch: what is still pending goes out once the own stream has drained (the last own backward
        is what the stages in front are waiting for; nothing may share the GPU with it)."""
        if self._rc_pending and self._own_tail is not None:
            self._own_tail.synchronize()
        while self._rc_pending:
            self._rc_issue_oldest()

    def _loss_head(self, buffer_id, stage_id, out):
        """Loss of one micro-batch on the last stage and its gradient scaled by 1 / micro_batches
        (reference engine.py:1649-1663, deepspeed/runtime/engine.py:1430-1431)."""
        labels = self.pipe_buffers["label"][buffer_id]
        if labels is None:
            raise PipelineError(f"ForwardPass({buffer_id}, {stage_id}): the last stage has no labels for this micro-batch")
        if labels.numel() != out.numel():
            raise PipelineError(f"labels of micro-batch {buffer_id} have {labels.numel()} elements, the last stage's output {out.numel()}")
        if self._loss_grad is None or self._loss_grad.shape != out.shape:
            self._loss_grad = torch.empty(tuple(out.shape), dtype=self.module.dtype, device=self.device)
            self._loss_ws = torch.empty(hip.mse_workspace(), dtype=torch.float32, device=self.device)
        self.module.loss_fn(out, labels, self._loss_grad, 1.0 / self.micro_batches, self.total_loss, True,
                            self._loss_ws, stream=self.main_stream)
        self.grad_layer[stage_id] = self._loss_grad
        self._loss_done.add((stage_id, buffer_id))

    def _exec_backward_pass(self, buffer_id, stage_id):
        grad = self.grad_layer.get(stage_id)
        if grad is None:
            raise PipelineError(f"BackwardPass({buffer_id}, {stage_id}) without a received gradient")
        self.ctx.key_len = self.queue.key_len(buffer_id)
        self.ctx.dropout_base = (self.module.base_seed, self.global_steps, buffer_id)
        dst = self._input_grad_store[stage_id][buffer_id]
        kl = self.ctx.key_len
        deferred = self._deferred.get((stage_id, buffer_id), False)
        key = ("B", stage_id, buffer_id, id(self.ctx), grad.data_ptr(), dst.data_ptr(),
               None if kl is None else kl.data_ptr(), deferred)
        self._graphed(key, self.ctx.stream, lambda: self.module.backward(grad, dst, stage_id, slot=buffer_id, ctx=self.ctx,
                                                                         deferred=deferred))
        key = f"input_grad_{stage_id}"
        if key in self.pipe_buffers:
            self.pipe_buffers[key][buffer_id] = dst
        self.grad_layer[stage_id] = None
        if hasattr(self.queue, "note_done"):
            self.queue.note_done("B", buffer_id, stage_id, self.main_stream)
        if self.rc_issue == "bubble":
            self._mark_own_tail()

    def _exec_reduce_grads(self, stage_id):
        # data-parallel world of one: the all-reduce of deepspeed/runtime/engine.py:1773-1802 is the identity
        return

    def _exec_optimizer_step(self):
        if self.config.gradient_clipping > 0.0 and hasattr(self.optimizer, "clip_coef"):
            # clip_fp32_gradients of the reference (deepspeed/runtime/engine.py:1521-1531): the norm and the
            # coefficient stay on the device, the Adam kernel scales the gradients as it reads them
            self.grad_norm = self.optimizer.clip_coef(self.config.gradient_clipping, stream=self.main_stream)
            self.optimizer.step(stream=self.main_stream, grad_scale=self.grad_norm[1:])
        else:
            self.optimizer.step(stream=self.main_stream)
        if self.lr_scheduler is not None:
            self.lr_scheduler.step()
        self.global_steps += 1
        self.global_samples += self.train_batch_size()

    def _exec_send_weights(self, stage_id):
        """Publish the parameters and Adam moments of ``stage_id`` for the stage that shadows it
        (reference engine.py:2084-2108, never wired there).  A stage is one flat arena per kind, so
        the message is four tensors; on one GPU the link hands over references."""
        if not hasattr(self.queue, "send_weights"):
            return
        sp = self.module.stage_params[stage_id]
        self.queue.send_weights(stage_id, {"master": sp.master, "exp_avg": sp.exp_avg, "exp_avg_sq": sp.exp_avg_sq,
                                           "step": self.optimizer.step_count(stage_id)})

    def _exec_recv_weights(self, stage_id):
        """Refresh the shadow copy of ``stage_id`` (reference engine.py:2110-2137): device-to-device
        copies into the arenas that were allocated when the shadow stage was built."""
        if not hasattr(self.queue, "recv_weights") or stage_id not in self.r_stage_ids:
            return
        msg = self.queue.recv_weights(stage_id)
        if msg is None:
            return
        if not self.eager_recovery:
            # lazy mode keeps host mirrors only (engine.py:336-350): parameters and both moments come
            # down as three flat copies and are scattered into the named buffers
            names = self.module.param_name_buckets[stage_id]
            pflat = getattr(self.param_buffers[stage_id], "flat", None)
            sflat = getattr(self.state_buffers[stage_id], "flat", None)
            if pflat is not None and sflat is not None and pflat.numel() == msg["master"].numel():
                pflat.copy_(msg["master"])                   # the named buffers are views of these three
                sflat["exp_avg"].copy_(msg["exp_avg"])
                sflat["exp_avg_sq"].copy_(msg["exp_avg_sq"])
                self._shadow_step = msg["step"]
                return
            host = {k: msg[k].cpu() for k in ("master", "exp_avg", "exp_avg_sq")}
            off = 0
            for i, name in enumerate(names):
                buf = self.param_buffers[stage_id][name]
                n = buf.numel()
                buf.copy_(host["master"][off: off + n].view_as(buf))
                self.state_buffers[stage_id][f"{i}.exp_avg"].copy_(host["exp_avg"][off: off + n].view_as(buf))
                self.state_buffers[stage_id][f"{i}.exp_avg_sq"].copy_(host["exp_avg_sq"][off: off + n].view_as(buf))
                off += n
            self._shadow_step = msg["step"]
            return
        sp = self.module.stage_params[stage_id]
        sp.master.copy_(msg["master"])
        sp.exp_avg.copy_(msg["exp_avg"])
        sp.exp_avg_sq.copy_(msg["exp_avg_sq"])
        sp.refresh_compute()
        self._shadow_step = msg["step"]

    # ------------------------------------------------------------------ moving layers (reconfiguration)
    def _stage_of_layer(self, layer_idx):
        for sid in self.module.stage_params:
            if self.module.parts[sid] <= layer_idx < self.module.parts[sid + 1]:
                return sid
        raise PipelineError(f"layer {layer_idx} is not built in this process")

    def get_layer_state(self, layer_idxs):
        """``{idx: [state_dict, [ {exp_avg, exp_avg_sq} per parameter ]]}``: the ``state`` argument of
        ``send_layers`` (reference engine.py:893-901, ``get_optimizer_state`` :1005-1014)."""
        out = {}
        for idx in layer_idxs:
            sd = self.module.layer_state_dict(idx)
            m, v = self.module.layer_state_dict(idx, "exp_avg"), self.module.layer_state_dict(idx, "exp_avg_sq")
            out[idx] = [sd, [{"exp_avg": m[name], "exp_avg_sq": v[name]} for name in sd]]
        return out

    def send_layers(self, dst_rank, layer_idxs, state):
        """Layers and their Adam moments as the reference's two flat tensors (engine.py:893-927).
        Returns them; a fabric that can carry them also gets them handed over."""
        from .wire import pack_layers
        layer_tensor, optim_tensor = pack_layers(layer_idxs, state)
        if hasattr(self.queue, "send_layer_tensors"):
            self.queue.send_layer_tensors(dst_rank, layer_tensor, optim_tensor)
        return layer_tensor, optim_tensor

    def recv_layers(self, src_rank, layer_idxs, tensors=None):
        """Inverse of :meth:`send_layers` (engine.py:929-1003): ``recvd_state`` keyed by layer index.
        Shapes come from this process's own layer specs, as in the reference."""
        from .wire import unpack_layers
        if tensors is None:
            tensors = self.queue.recv_layer_tensors(src_rank)
        shapes = {}
        for idx in layer_idxs:
            sd = self.module.layer_state_dict(idx)
            shapes[idx] = OrderedDict((k, tuple(v.shape)) for k, v in sd.items())
        return unpack_layers(layer_idxs, shapes, tensors[0], tensors[1])

    def load_layer_state(self, recvd_state):
        """Put received layers (parameters and moments) into this process's arenas."""
        for idx, (sd, opt) in recvd_state.items():
            sp = self.module.stage_params[self._stage_of_layer(idx)]
            for (name, t), moments in zip(sd.items(), opt):
                self.module.load_layer_tensor(idx, name, t)
                self.module.load_layer_tensor(idx, name, moments["exp_avg"], "exp_avg")
                self.module.load_layer_tensor(idx, name, moments["exp_avg_sq"], "exp_avg_sq")
            sp.refresh_compute()

    _INSTRUCTION_MAP = {
        schedule.OptimizerStep: _exec_optimizer_step,
        schedule.ReduceGrads: _exec_reduce_grads,
        schedule.LoadMicroBatch: _exec_load_micro_batch,
        schedule.ForwardPass: _exec_forward_pass,
        schedule.BackwardPass: _exec_backward_pass,
        schedule.SendActivation: _exec_send_activations,
        schedule.RecvActivation: _exec_recv_activations,
        schedule.SendGrad: _exec_send_grads,
        schedule.RecvGrad: _exec_recv_grads,
        schedule.SendWeights: _exec_send_weights,
        schedule.RecvWeights: _exec_recv_weights,
    }

    def _exec_schedule(self, pipe_schedule):
        """Interpreter loop (reference engine.py:2339-2394): returns None, or ``(step, exception)``
        when a neighbour failed."""
        self._reserve_pipe_buffers(pipe_schedule.num_pipe_buffers())
        for step_i, step_cmds in enumerate(pipe_schedule):
            if getattr(self, "_replay_until", None) == step_i and self.last_failover and "t_detect" in self.last_failover:
                # the successor's lost work has been redone: the stage is back where it was when the
                # failure was detected (pause = detection -> here, GPU drained)
                torch.cuda.synchronize(self.device)
                self.last_failover["pause_s"] = time.perf_counter() - self.last_failover["t_detect"]
                self._replay_until = None
            if self._debug:
                self.log(f"step {step_i}: {step_cmds}")
            try:
                for cmd in step_cmds:
                    handler = self._INSTRUCTION_MAP.get(type(cmd))
                    if handler is None:
                        raise RuntimeError(f"{self.__class__.__name__} does not understand instruction {cmd!r}")
                    handler(self, **cmd.kwargs)
            except (NextStageException, PrevStageException, AllReduceException) as e:
                return step_i, e
        return None
