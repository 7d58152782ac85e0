"""Wire format of whole layers and the per-layer checkpoint files (CPU)."""
from collections import OrderedDict

import numpy as np
import pytest
import torch

from bamboo_amd import wire
from oracle import wire as owire


def make_state():
    # layer 3: w [2,3], b [3]; layer 5: g [4]
    def t(start, shape):
        n = int(np.prod(shape))
        return torch.arange(start, start + n, dtype=torch.float32).view(shape)
    s3 = OrderedDict(w=t(0, (2, 3)), b=t(10, (3,)))
    s5 = OrderedDict(g=t(20, (4,)))
    o3 = [{"exp_avg": t(100, (2, 3)), "exp_avg_sq": t(200, (2, 3))}, {"exp_avg": t(110, (3,)), "exp_avg_sq": t(210, (3,))}]
    o5 = [{"exp_avg": t(120, (4,)), "exp_avg_sq": t(220, (4,))}]
    return {3: [s3, o3], 5: [s5, o5]}


def test_known_answer():
    lt, ot = wire.pack_layers([3, 5], make_state())
    assert lt.tolist() == [0, 1, 2, 3, 4, 5, 10, 11, 12, 20, 21, 22, 23]
    assert ot.tolist() == ([100, 101, 102, 103, 104, 105, 200, 201, 202, 203, 204, 205] +
                           [110, 111, 112, 210, 211, 212] + [120, 121, 122, 123, 220, 221, 222, 223])
    # the order of the index list is the order on the wire
    lt2, _ = wire.pack_layers([5, 3], make_state())
    assert lt2.tolist()[:4] == [20, 21, 22, 23]
    # oracle restatement agrees
    st = make_state()
    nstate = {i: [{k: v.numpy() for k, v in sd.items()}, [{k: v.numpy() for k, v in e.items()} for e in opt]]
              for i, (sd, opt) in st.items()}
    olt, oot = owire.pack_layers([3, 5], nstate)
    assert olt.tolist() == lt.tolist() and oot.tolist() == ot.tolist()


def test_round_trip_and_errors():
    st = make_state()
    shapes = {i: OrderedDict((k, tuple(v.shape)) for k, v in sd.items()) for i, (sd, _) in st.items()}
    lt, ot = wire.pack_layers([3, 5], st)
    back = wire.unpack_layers([3, 5], shapes, lt, ot)
    oback = owire.unpack_layers([3, 5], shapes, lt.numpy(), ot.numpy())
    for i in (3, 5):
        for (k, v), e, e0 in zip(st[i][0].items(), back[i][1], st[i][1]):
            assert torch.equal(back[i][0][k], v)
            assert np.array_equal(oback[i][0][k], v.numpy())
            assert torch.equal(e["exp_avg"], e0["exp_avg"]) and torch.equal(e["exp_avg_sq"], e0["exp_avg_sq"])
        for e, oe in zip(back[i][1], oback[i][1]):
            assert np.array_equal(oe["exp_avg_sq"], e["exp_avg_sq"].numpy())
    with pytest.raises(ValueError):
        wire.unpack_layers([3], shapes, lt, ot)            # left-over elements
    bad = make_state()
    bad[3][1].pop()
    with pytest.raises(ValueError):
        wire.pack_layers([3], bad)
    assert wire.pack_layers([], {})[0].numel() == 0
    assert wire.ckpt_layer_path("/x", 7).endswith("layer_07-model_states.pt")
