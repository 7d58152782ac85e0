"""Engine configuration: the subset of the DeepSpeed JSON the pipeline path reads.

Batch triad ``train_batch_size = micro_batch * gradient_accumulation_steps * dp_world``
as in ``deepspeed/runtime/config.py:862-932`` (any two determine the third; dp_world is 1
here), ``optimizer{type, params{lr, betas, eps, weight_decay}}``, ``gradient_clipping``, ``steps_per_print``,
``wall_clock_breakdown`` (``DeepSpeedExamples/pipeline_parallelism/transformer.json:1-17``).
``bf16.enabled`` selects bf16 compute with fp32 master weights (this build's analogue of the
reference's fp16 wrapper, ``deepspeed/runtime/fp16/fused_optimizer.py:24-122``).
"""
import json

import torch


class BambooConfig:
    def __init__(self, config=None, dp_world_size=1):
        if config is None:
            config = {}
        if isinstance(config, str):
            with open(config) as f:
                config = json.load(f)
        self.raw = dict(config)
        tb = config.get("train_batch_size")
        mb = config.get("train_micro_batch_size_per_gpu")
        gas = config.get("gradient_accumulation_steps")
        if tb is not None and mb is not None and gas is None:
            gas = tb // (mb * dp_world_size)
        elif tb is not None and gas is not None and mb is None:
            mb = tb // (gas * dp_world_size)
        elif mb is not None and gas is not None and tb is None:
            tb = mb * gas * dp_world_size
        elif tb is not None and mb is None and gas is None:
            gas, mb = 1, tb // dp_world_size
        elif mb is not None and tb is None and gas is None:
            gas, tb = 1, mb * dp_world_size
        if tb is None or mb is None or gas is None:
            raise ValueError("config needs train_batch_size and/or train_micro_batch_size_per_gpu")
        if tb != mb * gas * dp_world_size or min(tb, mb, gas) <= 0:
            raise ValueError(f"train_batch_size ({tb}) != micro_batch ({mb}) * grad_acc ({gas}) * dp ({dp_world_size})")
        self.train_batch_size, self.train_micro_batch_size_per_gpu, self.gradient_accumulation_steps = tb, mb, gas

        opt = config.get("optimizer", {"type": "Adam", "params": {}})
        self.optimizer_name = opt.get("type", "Adam")
        if self.optimizer_name.lower() not in ("adam", "adamw"):
            raise ValueError(f"optimizer {self.optimizer_name!r} is not supported by the fused HIP Adam")
        p = opt.get("params", {})
        self.lr = float(p.get("lr", 1e-3))
        self.betas = tuple(p.get("betas", (0.9, 0.999)))
        self.eps = float(p.get("eps", 1e-8))
        self.weight_decay = float(p.get("weight_decay", 0.0))
        self.bias_correction = bool(p.get("bias_correction", True))
        # reference default: Adam type => adam_w_mode unless torch_adam (deepspeed/runtime/engine.py:985-1008)
        self.adam_w_mode = bool(p.get("adam_w_mode", True))
        # clip the global gradient norm to this value before the optimizer step; 0 = off
        # (deepspeed/runtime/config.py "gradient_clipping", used in _take_model_step, deepspeed/runtime/engine.py:1526-1531)
        self.gradient_clipping = float(config.get("gradient_clipping", 0.0))
        if self.gradient_clipping < 0:
            raise ValueError("gradient_clipping must be >= 0")
        self.steps_per_print = int(config.get("steps_per_print", 10))
        self.wall_clock_breakdown = bool(config.get("wall_clock_breakdown", False))
        self.bf16 = bool(config.get("bf16", {}).get("enabled", False))
        if config.get("fp16", {}).get("enabled", False):
            raise ValueError("fp16 is not implemented; use bf16.enabled or fp32")

    @property
    def compute_dtype(self):
        return torch.bfloat16 if self.bf16 else torch.float32
