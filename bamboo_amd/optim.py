"""Fused Adam over the flat parameter arenas of the stages a process executes.

Host side of the reference's ``FusedAdam`` (deepspeed/ops/adam/fused_adam.py:85-182): one
``step`` counter per group, moments start at zero, ``adam_w_mode`` selects decoupled weight
decay, one multi-tensor launch per step.  Because a stage's parameters are one contiguous
fp32 arena (with fp32 gradient, ``exp_avg``, ``exp_avg_sq`` arenas of the same layout and an
optional bf16 compute copy), the tensor list handed to ``bb_adam_multi`` has one entry per
stage; the kernel writes the bf16 copy and clears the gradient in the same pass, which is
the engine's ``zero_grad`` (deepspeed/runtime/engine.py:1550-1554).
"""
from collections import OrderedDict

from . import hip


class FusedAdam:
    def __init__(self, params=None, lr=1e-3, bias_correction=True, betas=(0.9, 0.999), eps=1e-8,
                 adam_w_mode=True, weight_decay=0.0, amsgrad=False, set_grad_none=True):
        if amsgrad:
            raise RuntimeError("FusedAdam does not support the AMSGrad variant.")
        self.defaults = dict(lr=lr, bias_correction=bias_correction, betas=betas, eps=eps, weight_decay=weight_decay)
        self.param_groups = [dict(self.defaults, params=[])]
        self.adam_w_mode = 1 if adam_w_mode else 0
        self.stages = OrderedDict()   # stage_id -> StageParams

    def add_stage(self, stage_id, stage_params):
        """Put the parameters of a (newly owned) stage under this optimizer; its moment arenas
        were allocated with the stage, so nothing is allocated here."""
        if stage_id not in self.stages:
            self.stages[stage_id] = stage_params
            self.param_groups[0]["params"].append(stage_params.master)

    @property
    def state(self):
        return {sid: {"exp_avg": sp.exp_avg, "exp_avg_sq": sp.exp_avg_sq} for sid, sp in self.stages.items()}

    def step_count(self, stage_id=None):
        """Steps taken so far (one counter for the group, as in the reference: every stage of a
        pipeline steps once per batch, so an absorbed stage continues with the same count)."""
        return self.param_groups[0].get("step", 0)

    def zero_grad(self):
        for sp in self.stages.values():
            sp.grad.zero_()

    def clip_coef(self, max_norm, stream=None):
        """Global-norm clipping over the gradients of every stage under this optimizer (the reference clips what
        ``module.parameters()`` yields with a gradient: own stage, and an absorbed one after a failover;
        deepspeed/runtime/engine.py:1521-1531): returns a device tensor ``[norm, coefficient]``; hand
        ``[1:]`` to :meth:`step` as ``grad_scale``."""
        grads = [sp.grad for sp in self.stages.values()]
        need = hip.grad_clip_workspace(grads)
        if getattr(self, "_clip_ws", None) is None or self._clip_ws.numel() < need:
            import torch
            self._clip_ws = torch.empty(need, dtype=torch.float32, device=grads[0].device)
            self._clip_out = torch.zeros(2, dtype=torch.float32, device=grads[0].device)
        hip.grad_clip_coef(grads, max_norm, self._clip_out, self._clip_ws, stream=stream)
        return self._clip_out

    def step(self, closure=None, stream=None, grad_scale=None):
        group = self.param_groups[0]
        group["step"] = group.get("step", 0) + 1
        sps = list(self.stages.values())
        lowp = [sp.compute if sp.compute is not sp.master else None for sp in sps]
        hip.adam_multi([sp.grad for sp in sps], [sp.master for sp in sps], [sp.exp_avg for sp in sps],
                       [sp.exp_avg_sq for sp in sps], lowp if any(t is not None for t in lowp) else None,
                       lr=group["lr"], beta1=group["betas"][0], beta2=group["betas"][1], eps=group["eps"],
                       step=group["step"], adam_w_mode=bool(self.adam_w_mode),
                       bias_correction=group["bias_correction"], weight_decay=group["weight_decay"],
                       zero_grad=True, grad_scale=grad_scale, stream=stream)
        return None
