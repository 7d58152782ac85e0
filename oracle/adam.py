"""Fused-Adam update formula (TEST ORACLE).

Follows csrc/adam/multi_tensor_adam.cu:84-108 (per-element update, fp32 maths) and
:138-142 (bias corrections computed on the host) and the host loop of
deepspeed/ops/adam/fused_adam.py:85-182 (one shared ``step`` counter per group,
moments start at zero, ``adam_w_mode`` selects decoupled weight decay)."""
import numpy as np


def adam_step(p, g, m, v, step, lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8,
              weight_decay=0.0, adam_w_mode=True, bias_correction=True):
    """In-place update of fp32 numpy arrays p, m, v given gradient g."""
    f = np.float32
    p32, g32 = p.astype(f, copy=False), g.astype(f, copy=True)
    # the betas are C floats in the reference; the power is taken in double (std::pow(float, int))
    bc1 = f(1.0 - float(f(beta1)) ** step) if bias_correction else f(1.0)
    bc2 = f(1.0 - float(f(beta2)) ** step) if bias_correction else f(1.0)
    b1, b2, lr, eps, wd = f(beta1), f(beta2), f(lr), f(eps), f(weight_decay)
    if not adam_w_mode:
        g32 = g32 + wd * p32
    m[...] = b1 * m + (f(1.0) - b1) * g32
    v[...] = b2 * v + (f(1.0) - b2) * g32 * g32
    update = (m / bc1) / (np.sqrt(v / bc2) + eps)
    if adam_w_mode:
        update = update + wd * p32
    p[...] = p32 - lr * update
    return p, m, v


def clip_grad_norm(grads, max_norm):
    """Global-norm clipping of a list of fp32 gradient arrays, in place; returns (total_norm, clip_coef).

    Follows clip_grad_norm_ (deepspeed/runtime/utils.py:295-326) as _take_model_step calls it for fp32
    gradients (deepspeed/runtime/engine.py:1521-1531), norm_type 2, one process: total_norm = (sum over the
    tensors of ||g||_2 ** 2) ** 0.5, summed in Python floats; clip_coef = max_norm / (total_norm + 1e-6); the
    gradients are multiplied by it (in fp32) only when it is below 1."""
    total = 0.0
    for g in grads:
        total += float(np.sqrt(np.sum(g.astype(np.float64) ** 2))) ** 2
    total_norm = total ** 0.5
    clip_coef = float(max_norm) / (total_norm + 1e-6)
    if clip_coef < 1:
        for g in grads:
            g *= np.float32(clip_coef)
    return total_norm, clip_coef
