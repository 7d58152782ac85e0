"""A whole Bamboo pipeline in one process on one GPU: one :class:`PipelineEngine` per stage, each
running ``train_batch`` in its own thread, connected by a :class:`LocalFabric`.

This is the caller's side of the single-stage path: the stages around the one that is lost.  It
exists to exercise the reference's three-party failure protocol end to end (engine.py:1190-1303) --
the predecessor of the lost stage promotes its shadow layers and replays the lost work
(``NextStageFailoverSchedule``), the successor re-sends the gradients the lost stage had been given
(``PrevStageFailoverSchedule``), both agree on the failed step -- and the shadow-weight refresh
that keeps redundant forwards meaningful after optimizer steps (engine.py:2084-2137).  Every
engine issues its kernels to the same stream of the one GPU, so the stages time-share it: this
is a functional harness, not a throughput configuration.
"""
import itertools
import threading

from . import initialize
from .module import PipelineModule
from .p2p import LocalFabric, StageKilled


class _Cycle:
    """Training data for LoadMicroBatch: the given (input, label) micro-batches, repeated forever;
    every engine iterates its own copy."""

    def __init__(self, micro_batches):
        self.micro_batches = list(micro_batches)

    def __iter__(self):
        return itertools.cycle(self.micro_batches)


class LocalPipeline:
    def __init__(self, layers, num_stages, config, shape, dtype, micro_batches, loss_fn, redundancy_level=1,
                 eager_recovery=True, rc_stream=False, device="cuda:0", partition_method="uniform",
                 custom_partitions=(), timeout=120.0):
        """layers: layer specs of the whole model; shape: ``(micro_batch, seq, hidden)`` of the
        activations between stages; micro_batches: list of ``(input, label)`` tensors of one batch
        (used again for every batch); loss_fn: loss of the last stage (``bamboo_amd.MSELoss()``)."""
        self.num_stages = num_stages
        M = config["gradient_accumulation_steps"]
        if len(micro_batches) != M:
            raise ValueError(f"need {M} micro-batches of data, got {len(micro_batches)}")
        self.fabric = LocalFabric(num_stages, shape, dtype, M, device=device, timeout=timeout)
        self.engines = {}
        for s in range(num_stages):
            model = PipelineModule(list(layers), num_stages=num_stages, partition_method=partition_method,
                                   custom_partitions=list(custom_partitions), stage_id=s, dtype=dtype, device=device,
                                   loss_fn=loss_fn)
            engine, _, _, _ = initialize(model=model, config=config, training_data=_Cycle(micro_batches),
                                         redundancy_level=redundancy_level, eager_recovery=eager_recovery,
                                         activation_queue=self.fabric.endpoint(s), rc_stream=rc_stream,
                                         install_signal_handler=False)
            self.engines[s] = engine
        self.lost = []
        if not eager_recovery:
            # lazy mode starts from zero host mirrors (reference module.py:229-260): fill them once
            self.sync_shadow_weights()

    def engine_of(self, stage_id):
        """The engine that currently runs ``stage_id`` (its own, or the predecessor that absorbed it)."""
        for e in self.engines.values():
            if stage_id in e.stage_ids:
                return e
        raise KeyError(stage_id)

    def kill(self, stage_id, at_micro_batch=0):
        """Preempt the engine of ``stage_id`` during the next batch."""
        self.fabric.kill(stage_id, at_micro_batch)

    def train_batch(self, sync_weights=True):
        """One batch on every live engine; returns the loss seen by the last stage."""
        results, errors = {}, {}

        def run(s, engine):
            try:
                results[s] = engine.train_batch()
            except StageKilled:
                results[s] = None
            except BaseException as e:  # noqa: BLE001 - re-raised in the caller's thread
                errors[s] = e

        threads = [threading.Thread(target=run, args=(s, e), name=f"stage{s}", daemon=True)
                   for s, e in self.engines.items()]
        for t in threads:
            t.start()
        for t in threads:
            t.join()
        if errors:
            s, e = sorted(errors.items())[0]
            raise RuntimeError(f"stage {s} failed: {e!r}") from e
        for s in [s for s, r in results.items() if r is None]:
            self.lost.append(s)
            del self.engines[s]
        if sync_weights:
            self.sync_shadow_weights()
        return results[max(self.engines)]

    def sync_shadow_weights(self):
        """After the optimizer steps: every stage publishes its parameters and Adam moments, every
        engine refreshes the shadow copy it keeps of its successor (SendWeights / RecvWeights)."""
        for e in self.engines.values():
            for sid in e.stage_ids:
                e._exec_send_weights(sid)
        for e in self.engines.values():
            for sid in e.r_stage_ids:
                e._exec_recv_weights(sid)
