"""Flat wire format of whole layers (TEST INFRASTRUCTURE ONLY), restated with numpy from
``PipelineEngine.send_layers / recv_layers`` (deepspeed/runtime/pipe/engine.py:893-1003).

Pinned by a hand-written known answer (tests/test_wire.py): two layers, parameters of different
shapes, every element a distinct number, so a wrong order of layers, parameters or moments, or a
transposed reshape, changes the expected vector."""
import numpy as np


def pack_layers(layer_idxs, state):
    """state[idx] = [ordered {name: array}, [ {"exp_avg": a, "exp_avg_sq": a} per parameter ]]."""
    layer, optim = [], []
    for idx in layer_idxs:                               # engine.py:905-915
        sd, opt = state[idx]
        for v in sd.values():
            layer.append(np.asarray(v, dtype=np.float32).reshape(-1))
        for entry in opt:
            for v in entry.values():                     # dict order: exp_avg, exp_avg_sq
                optim.append(np.asarray(v, dtype=np.float32).reshape(-1))
    cat = lambda xs: np.concatenate(xs) if xs else np.zeros(0, np.float32)
    return cat(layer), cat(optim)


def unpack_layers(layer_idxs, layer_shapes, layer_vec, optim_vec):
    out, lo, oo = {}, 0, 0                               # engine.py:965-1001
    for idx in layer_idxs:
        sd = {}
        for name, shape in layer_shapes[idx].items():
            n = int(np.prod(shape))
            sd[name] = layer_vec[lo: lo + n].reshape(shape)
            lo += n
        out[idx] = [sd, []]
    for idx in layer_idxs:
        for name, shape in layer_shapes[idx].items():
            n = int(np.prod(shape))
            entry = {}
            for key in ("exp_avg", "exp_avg_sq"):
                entry[key] = optim_vec[oo: oo + n].reshape(shape)
                oo += n
            out[idx][1].append(entry)
    return out
