"""Interpreter of a stage's instruction stream over the oracle layers (TEST ORACLE, CPU).

Follows the reference engine's handlers (deepspeed/runtime/pipe/engine.py):
  RecvActivation  :1999-2041  local hand-off = detached clone with requires_grad, else recv
  ForwardPass     :1626-1678  module.forward(x, stage_id); result kept in output_{stage}[k];
                              early-out when the output already exists
  SendActivation  :1894-1933  skipped when the consumer stage is local
  RecvGrad        :2043-2082  local: grad of the consumer's input; else recv
  BackwardPass    :1680-1727  torch.autograd.backward(output, grad)
  SendGrad        :1935-1997
  OptimizerStep   :2139-2147 -> FusedAdam.step (deepspeed/ops/adam/fused_adam.py:85-182)
  last stage      :1649-1663  loss_model(outputs, labels) in the forward, backward of loss / GAS
and the failover branch of train_batch (:1190-1264): promote the shadow stage, run the
NextStageFailoverSchedule from step 0, one optimizer step for both stages.  The neighbours
are modelled exactly as the product's in-process queue models them: seeded activations in,
and either seeded output-gradients or an MSE loss head (gradient scaled by 1/micro_batches,
deepspeed/runtime/engine.py:1430-1431) out.
"""
import torch
import torch.nn.functional as F

from . import adam as oadam
from . import layers as olayers
from . import schedule as osched


class PeerFailure(Exception):
    pass


class OraclePeer:
    """Neighbour model: ``grads[stage][k]`` tensors (queue mode) or ``targets[stage][k]`` (mse)."""

    def __init__(self, activations, micro_batches, grads=None, targets=None, key_lens=None, labels=None):
        self.activations, self.M = activations, micro_batches
        self.grads, self.targets, self.key_lens = grads or {}, targets or {}, key_lens
        self.relu_masks = {}      # (stage, k) -> per-layer ReLU decisions of the run the oracle is compared with
        self.labels = labels      # labels[k] of the last stage's own loss (LoadMicroBatch), if this process hosts it
        self.loss = 0.0
        self.dead_from, self.dead_stage = None, None
        self._mse_grads = {}

    def check(self, k, stage):
        if self.dead_from is not None and stage == self.dead_stage and k >= self.dead_from:
            raise PeerFailure()

    def send_activation(self, k, out, stage):
        self.check(k, stage)
        if stage in self.targets:
            o = out.detach().clone().requires_grad_(True)
            loss = F.mse_loss(o, self.targets[stage][k].view_as(o))
            self.loss = self.loss + loss.detach()
            (loss / self.M).backward()
            self._mse_grads[(stage, k)] = o.grad

    def recv_grad(self, k, stage):
        self.check(k, stage)
        if stage in self.targets:
            return self._mse_grads[(stage, k)]
        return self.grads[stage][k]


class OracleStage:
    def __init__(self, cfg, parts, stage_id, micro_batches, base_seed=1234, dtype=torch.float32,
                 redundancy_level=0, eager=False, adam=None, tail=False):
        """``tail``: the model ends with the reference script's two extra layers (final LayerNorm, sum over the hidden
        dimension; transformer.py:250): ``parts[-1]`` then counts them, and the last stage applies them."""
        self.tail = tail
        # a list of BottleneckCfg gives every block of the model its own shape (down-sampling / widening blocks)
        self.layer_cfgs = list(cfg) if isinstance(cfg, (list, tuple)) else None
        if self.layer_cfgs is not None:
            cfg = self.layer_cfgs[0]
        self.cfg, self.parts, self.stage_id, self.M = cfg, parts, stage_id, micro_batches
        self.S = len(parts) - 1
        self.dtype = dtype
        self.stage_ids = [stage_id]
        self.r_stage_ids = osched.redundant_stage_ids(redundancy_level, stage_id, self.S)
        self.eager = eager
        self.params = {}
        self.base_seed = base_seed
        self.build(stage_id)
        if eager:
            for r in self.r_stage_ids:
                self.build(r)
        self.adam = dict(lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.0, adam_w_mode=True)
        self.adam.update(adam or {})
        self.adam_state = {}
        self.step_count = 0

    def block_cfg(self, layer_idx):
        return self.cfg if self.layer_cfgs is None else self.layer_cfgs[layer_idx]

    def build(self, stage):
        conv = isinstance(self.cfg, olayers.BottleneckCfg)
        layers = []
        n_blocks = self.parts[-1] - (2 if self.tail else 0)
        for li in range(self.parts[stage], self.parts[stage + 1]):
            if li == n_blocks:            # the final LayerNorm: gain 1, shift 0
                h = self.cfg.hidden
                layers.append({"a_2": torch.ones(h, dtype=self.dtype).requires_grad_(True),
                               "b_2": torch.zeros(h, dtype=self.dtype).requires_grad_(True)})
                continue
            if li > n_blocks:             # x.sum(-1): no parameters
                layers.append({})
                continue
            if conv:
                p = olayers.init_bottleneck_params(self.block_cfg(li), self.base_seed + li, dtype=self.dtype)
            else:
                p = olayers.init_params(self.cfg, self.base_seed + li, dtype=self.dtype)
            layers.append({k: v.requires_grad_(True) for k, v in p.items()})
        self.params[stage] = layers

    def forward(self, x, stage, key_lens=None, relu_masks=None, drop_id=None):
        """``relu_masks``: per layer of the stage, the ReLU decisions to use (``oracle.layers.activation``):
        one tensor [batch, seq, ffn] per transformer layer, three NCHW tensors per bottleneck block."""
        masks = relu_masks if relu_masks is not None else [None] * len(self.params[stage])
        if isinstance(self.cfg, olayers.BottleneckCfg):
            # activations travel as [batch, H*W, C] (NHWC); torch convolutions want NCHW
            b, hw, c = x.shape
            side = int(round(hw ** 0.5))
            y = x.view(b, side, side, c).permute(0, 3, 1, 2)
            for li, (p, m) in enumerate(zip(self.params[stage], masks)):
                y = olayers.bottleneck(y, p, self.block_cfg(self.parts[stage] + li), m)
            return y.permute(0, 2, 3, 1).reshape(b, -1, y.shape[1])
        for li, (p, m) in enumerate(zip(self.params[stage], masks)):
            if set(p) == {"a_2", "b_2"}:
                x = olayers.script_tail(x, p, self.cfg.ln, self.cfg.eps)
            elif p:
                dm = None
                if getattr(self.cfg, "dropout", 0.0) > 0 and drop_id is not None:
                    # drop_id = (step, micro-batch): with the model's base seed and the layer's global index it names
                    # the masks, the same for a redundant forward, a normal one and a replay
                    dm = olayers.layer_drop_masks(self.cfg, self.base_seed, drop_id[0], drop_id[1], self.parts[stage] + li,
                                                  x.shape[0], x.shape[1])
                x = olayers.transformer_layer(x, p, self.cfg, key_lens, m, dm)
        return x

    def named_grads(self, stage):
        out = {}
        for li, p in enumerate(self.params[stage]):
            for k, v in p.items():
                out[f"{self.parts[stage] + li}.{k}"] = v.grad
        return out

    def named_params(self, stage):
        out = {}
        for li, p in enumerate(self.params[stage]):
            for k, v in p.items():
                out[f"{self.parts[stage] + li}.{k}"] = v
        return out

    # ------------------------------------------------------------------ interpreter
    def _exec(self, steps, peer, bufs, start=0):
        for i, cmds in enumerate(steps):
            if i < start:
                continue
            try:
                for name, k, s in cmds:
                    getattr(self, "_" + name)(k, s, peer, bufs)
            except PeerFailure:
                return i
        return None

    def _LoadMicroBatch(self, k, s, peer, bufs):
        pass

    def _RecvActivation(self, k, s, peer, bufs):
        if bufs["in"].get((s, k)) is not None:
            return
        if s - 1 in self.stage_ids:
            x = bufs["out"][(s - 1, k)].detach().clone()
        else:
            x = peer.activations[k].detach().clone()
        bufs["in"][(s, k)] = x.requires_grad_(True)

    def _ForwardPass(self, k, s, peer, bufs):
        if bufs["out"].get((s, k)) is not None:
            if (s == self.S - 1 and peer.labels is not None and s in self.stage_ids
                    and (s, k) not in bufs.get("loss", {})):
                # replay after absorbing the last stage: the redundant forward left the output, the loss
                # is still to be computed
                out = bufs["out"][(s, k)]
                loss = F.mse_loss(out, peer.labels[k].view_as(out))
                bufs.setdefault("loss", {})[(s, k)] = loss
                peer.loss = peer.loss + loss.detach()
            return
        kl = None if peer.key_lens is None else peer.key_lens[k]
        out = self.forward(bufs["in"][(s, k)], s, kl, peer.relu_masks.get((s, k)), (self.step_count, k))
        bufs["out"][(s, k)] = out
        if s == self.S - 1 and peer.labels is not None and s in self.stage_ids:
            # last stage: loss_model(outputs, labels), summed into total_loss (engine.py:1649-1663); counted
            # once per micro-batch (the reference recomputes the forward of an absorbed last stage, whose
            # output it never keeps, :1646 -- same value)
            loss = F.mse_loss(out, peer.labels[k].view_as(out))
            bufs.setdefault("loss", {})[(s, k)] = loss
            peer.loss = peer.loss + loss.detach()

    def _SendActivation(self, k, s, peer, bufs):
        if s + 1 in self.stage_ids:
            return
        peer.send_activation(k, bufs["out"][(s, k)], s)

    def _RecvGrad(self, k, s, peer, bufs):
        if s + 1 in self.stage_ids:
            bufs["grad"][s] = bufs["in"][(s + 1, k)].grad
        else:
            bufs["grad"][s] = peer.recv_grad(k, s)

    def _BackwardPass(self, k, s, peer, bufs):
        if s == self.S - 1 and (s, k) in bufs.get("loss", {}):
            # loss / gradient_accumulation_steps, then backward (deepspeed/runtime/engine.py:1430-1431,1478)
            (bufs["loss"][(s, k)] / self.M).backward()
            return
        out = bufs["out"][(s, k)]
        torch.autograd.backward(out, bufs["grad"][s].view_as(out))

    def _SendGrad(self, k, s, peer, bufs):
        bufs["sent_grad"][(s, k)] = bufs["in"][(s, k)].grad

    def _ReduceGrads(self, k, s, peer, bufs):
        pass

    def _OptimizerStep(self, k, s, peer, bufs):
        self.step_count += 1
        for sid in self.stage_ids:
            for li, p in enumerate(self.params[sid]):
                for name, t in p.items():
                    key = (sid, li, name)
                    if key not in self.adam_state:
                        self.adam_state[key] = (torch.zeros_like(t).numpy(), torch.zeros_like(t).numpy())
                    m, v = self.adam_state[key]
                    g = t.grad if t.grad is not None else torch.zeros_like(t)
                    pn = t.detach().numpy()
                    oadam.adam_step(pn, g.numpy(), m, v, self.step_count, **self.adam)
                    t.grad = None

    def own_stream(self):
        own = osched.train_schedule(self.M, self.S, self.stage_id)
        if self.r_stage_ids and self.eager:
            return osched.eager_merge(own, osched.train_schedule(self.M, self.S, self.r_stage_ids[0]))
        return own

    def run_batch(self, peer, optimizer_step=True):
        """One batch.  Returns buffers (inputs, outputs, gradients) and failover info."""
        bufs = {"in": {}, "out": {}, "grad": {}, "sent_grad": {}}
        if len(self.stage_ids) == 2:
            steps = osched.next_stage_failover(osched.train_schedule(self.M, self.S, self.stage_ids[0]),
                                               osched.train_schedule(self.M, self.S, self.stage_ids[1]), 0, 0)
        else:
            steps = self.own_stream()
        if not optimizer_step:
            steps = [[c for c in cmds if c[0] != "OptimizerStep"] for cmds in steps]
        failed = self._exec(steps, peer, bufs)
        info = {"failed_step": failed}
        if failed is not None:
            # failed_step = 0: the in-process peer has seen nothing of the dead successor's
            # traffic, so the replay keeps the successor's sends (schedule.py:349-353, second case)
            nxt = self.r_stage_ids[0]
            if nxt not in self.params:
                self.build(nxt)
            self.stage_ids.append(nxt)
            self.r_stage_ids = []
            steps = osched.next_stage_failover(osched.train_schedule(self.M, self.S, self.stage_id),
                                               osched.train_schedule(self.M, self.S, nxt), 0, failed)
            if not optimizer_step:
                steps = [[c for c in cmds if c[0] != "OptimizerStep"] for cmds in steps]
            again = self._exec(steps, peer, bufs)
            assert again is None
        return bufs, info
