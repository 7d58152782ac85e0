"""Dropout without stored masks (CPU): the numpy restatement of the decision function against the library's own
host-side evaluation of it, its statistics, and the placement of the four dropout sites of an encoder layer
against the module form of the reference layer with the same masks."""
import numpy as np
import pytest
import torch

from oracle import dropout as od
from oracle import layers as ol


def test_decision_function_equals_the_library():
    from bamboo_amd import hip
    rng = np.random.default_rng(3)
    for _ in range(20):
        ident = [int(v) for v in rng.integers(0, 2 ** 31, 5)]
        k = od.key(*ident)
        assert k == hip.dropout_key(*ident)
        p = float(rng.choice([0.1, 0.5, 0.013, 0.9]))
        idx = np.concatenate([np.arange(40), rng.integers(0, 2 ** 40, 40)]).astype(np.uint64)     # past 2^32 too
        want = od.keep(p, k, idx)
        got = np.array([hip.dropout_keep(p, k, int(i)) for i in idx])
        assert np.array_equal(want, got)
    assert od.threshold(0.1) == round(float(np.float32(0.1)) * 2 ** 16) == 6554 and od.threshold(0.0) == 0 and od.threshold(1e-9) == 1
    # one hand-computed value of the finalizer (x ^= x >> 16; x *= 0x7feb352d; x ^= x >> 15; x *= 0x846ca68b; x ^= x >> 16)
    # pins the restatement independently of the library: key (0, 0), pair 1 -> mix32(1)
    x = 1
    x ^= x >> 16; x = (x * 0x7FEB352D) & 0xFFFFFFFF; x ^= x >> 15; x = (x * 0x846CA68B) & 0xFFFFFFFF; x ^= x >> 16
    assert int(od.pair_bits((0, 0), 1)) == x
    assert bool(od.keep(0.5, (0, 0), 2)) == ((x & 0xFFFF) >= 32768) and bool(od.keep(0.5, (0, 0), 3)) == ((x >> 16) >= 32768)
    # p = 0 keeps everything
    assert od.keep(0.0, (1, 2), np.arange(1000)).all()


@pytest.mark.parametrize("p", [0.1, 0.5])
def test_mask_statistics(p):
    n = 1 << 20
    a = od.mask(p, od.key(1234, 0, 0, 3, 1), (n,))
    b = od.mask(p, od.key(1234, 0, 1, 3, 1), (n,))        # next micro-batch
    c = od.mask(p, od.key(1234, 0, 0, 3, 2), (n,))        # another site of the same layer
    sigma = (p * (1 - p) / n) ** 0.5
    for m in (a, b, c):
        assert abs(m.mean() - (1 - p)) < 5 * sigma
    # different keys: independent decisions (agreement (1-p)^2 + p^2), and no drift along the index
    for x, y in ((a, b), (a, c), (b, c)):
        assert abs((x == y).mean() - ((1 - p) ** 2 + p ** 2)) < 6 * (0.25 / n) ** 0.5
    quarters = a.reshape(4, -1).mean(1)
    assert np.abs(quarters - (1 - p)).max() < 5 * 2 * sigma
    # neighbouring elements are uncorrelated, also the two that share one hash (its low and its high sixteen bits)
    assert abs(np.corrcoef(a[:-1], a[1:])[0, 1]) < 5 / n ** 0.5
    assert abs(np.corrcoef(a[0::2], a[1::2])[0, 1]) < 5 / (n / 2) ** 0.5


def test_dropout_sites_of_the_layer_match_the_module_form():
    """oracle.layers.transformer_layer with explicit masks against the stand-in of the reference's EncoderLayer whose
    four nn.Dropout modules are replaced by multiplications with the same masks (x * mask / (1 - p), what nn.Dropout
    computes in training mode): outputs and all gradients, fp64.  A mask applied at the wrong place, or a missing
    1 / (1 - p), fails this."""
    from tests.reference_shapes import RefEncoderLayer
    torch.manual_seed(4)
    hid, heads, ffn, b, s, p = 32, 4, 64, 2, 6, 0.25
    ref = RefEncoderLayer(hid, heads, ffn, p).double()
    cfg = ol.TransformerCfg(hidden=hid, heads=heads, ffn=ffn, dropout=p)
    masks = ol.layer_drop_masks(cfg, 99, 2, 1, 5, b, s)
    assert masks[0].shape == (b, heads, s, s) and 0 < float(masks[2].mean()) < 1

    class Fixed(torch.nn.Module):
        def __init__(self, m):
            super().__init__()
            self.m = m

        def forward(self, t):
            return t * self.m.view_as(t) / (1 - p)
    ref.self_attn.dropout = Fixed(masks[od.SITE_ATTENTION])
    ref.sublayer[0].dropout = Fixed(masks[od.SITE_SUBLAYER0])
    ref.feed_forward.dropout = Fixed(masks[od.SITE_FFN])
    ref.sublayer[1].dropout = Fixed(masks[od.SITE_SUBLAYER1])
    prm = {k: v.detach().clone().requires_grad_(True) for k, v in ref.named_parameters()}
    x = torch.randn(b, s, hid, dtype=torch.float64, requires_grad=True)
    xr = x.detach().clone().requires_grad_(True)
    y, yr = ol.transformer_layer(x, prm, cfg, drop_masks=masks), ref(xr)
    torch.testing.assert_close(y, yr, rtol=1e-11, atol=1e-12)
    dy = torch.randn_like(yr)
    y.backward(dy)
    yr.backward(dy)
    torch.testing.assert_close(x.grad, xr.grad, rtol=1e-10, atol=1e-12)
    for k, v in ref.named_parameters():
        torch.testing.assert_close(prm[k].grad, v.grad, rtol=1e-10, atol=1e-12, msg=k)
    # and the masks matter: without them the result differs
    assert not torch.allclose(ol.transformer_layer(x, prm, cfg), yr)
