"""Wire and file formats for moving layers between processes.

Reconfiguration in the reference ships whole layers with their optimizer state as two flat
tensors (``PipelineEngine.send_layers / recv_layers``, deepspeed/runtime/pipe/engine.py:893-1003):

  layer tensor   for each layer index in the list, its parameters in ``state_dict`` order,
                 flattened and concatenated;
  optim tensor   for each layer, for each parameter in the same order, ``exp_avg`` then
                 ``exp_avg_sq`` (FusedAdam keeps exactly these two per parameter), flattened and
                 concatenated.

The receiver knows the shapes from its own layer specs.  A layer's state is the pair
``[state_dict, [ {"exp_avg": t, "exp_avg_sq": t} per parameter ]]`` keyed by global layer index,
as in the reference.  Checkpoints are one file per layer, ``layer_XX-model_states.pt`` holding the
layer's ``state_dict`` (deepspeed/runtime/pipe/module.py:786-826).
"""
import os
from collections import OrderedDict

import torch

STATE_KEYS = ("exp_avg", "exp_avg_sq")


def flatten(tensors, dtype=torch.float32, device=None):
    """Concatenation of the flattened tensors (``_flatten_dense_tensors`` of the reference)."""
    if not tensors:
        return torch.empty(0, dtype=dtype, device=device)
    return torch.cat([t.reshape(-1).to(dtype) for t in tensors])


def unflatten(flat, shapes):
    """Views of ``flat`` with the given shapes, in order (``_unflatten_dense_tensors``)."""
    out, off = [], 0
    for shape in shapes:
        n = 1
        for d in shape:
            n *= d
        out.append(flat[off: off + n].view(shape))
        off += n
    if off != flat.numel():
        raise ValueError(f"flat tensor has {flat.numel()} elements, the shapes need {off}")
    return out


def pack_layers(layer_idxs, state):
    """``state[idx] = [state_dict, [optimizer dict per parameter]]`` -> (layer tensor, optim tensor)."""
    layer_bucket, optim_bucket = [], []
    for idx in layer_idxs:
        layer_state, optim_state = state[idx]
        layer_bucket.extend(layer_state.values())
        if len(optim_state) != len(layer_state):
            raise ValueError(f"layer {idx}: {len(layer_state)} parameters but {len(optim_state)} optimizer entries")
        for entry in optim_state:
            optim_bucket.extend(entry[k] for k in STATE_KEYS)
    return flatten(layer_bucket), flatten(optim_bucket)


def unpack_layers(layer_idxs, layer_shapes, layer_tensor, optim_tensor):
    """Inverse of :func:`pack_layers`; ``layer_shapes[idx]`` is an ordered ``{name: shape}``."""
    shapes = [shape for idx in layer_idxs for shape in layer_shapes[idx].values()]
    params = unflatten(layer_tensor, shapes)
    moments = unflatten(optim_tensor, [s for shape in shapes for s in (shape, shape)])
    out, pi = {}, 0
    for idx in layer_idxs:
        sd, opt = OrderedDict(), []
        for name in layer_shapes[idx]:
            sd[name] = params[pi]
            opt.append({STATE_KEYS[0]: moments[2 * pi], STATE_KEYS[1]: moments[2 * pi + 1]})
            pi += 1
        out[idx] = [sd, opt]
    return out


def ckpt_layer_path(ckpt_dir, layer_idx):
    return os.path.join(ckpt_dir, f"layer_{layer_idx:02d}-model_states.pt")
