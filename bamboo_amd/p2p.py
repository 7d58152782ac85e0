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
                 key_len_range=None):
        """shape: activation shape ``[micro_batch, seq, hidden]`` (same for every stage boundary);
        stage_ids: stages whose *outputs* this queue must answer for (own stage and, for failover,
        the shadowed stage)."""
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
            if grad_mode == "queue":
                self.grads[sid] = [self._randn(("grad", sid, k)) for k in range(micro_batches)]
            else:
                self.targets[sid] = [self._randn(("target", sid, k)) for k in range(micro_batches)]
                self.grads[sid] = [torch.zeros(self.shape, dtype=dtype, device=self.device) for _ in range(micro_batches)]

    _TAGS = {"act": 11, "grad": 23, "target": 37, "len": 41}

    def _tag_seed(self, tag):
        """Stable seed from (kind, ids...): independent of PYTHONHASHSEED."""
        h = self.seed
        for t in tag:
            h = (h * 1000003 + self._TAGS.get(t, t) + 7) % (2 ** 31 - 1)
        return h

    def _randn(self, tag):
        g = torch.Generator().manual_seed(self._tag_seed(tag))
        return torch.randn(self.shape, generator=g, dtype=torch.float32).to(self.dtype).to(self.device)

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

    def ping(self, stage_id):
        if self.dead_from is not None and stage_id == self.dead_stage and self.dead_from <= 0:
            raise NextStageException(f"successor of stage {stage_id} does not answer")
