"""Pins of the layer oracle against torch library routines and closed forms."""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import adam as oadam
from oracle import layers as ol


def test_annotated_layernorm_closed_form():
    torch.manual_seed(0)
    x = torch.randn(5, 7, 32, dtype=torch.float64)
    g, b = torch.randn(32, dtype=torch.float64), torch.randn(32, dtype=torch.float64)
    y = ol.layer_norm(x, g, b, "annotated", 1e-6)
    xn = x.numpy()
    mean = xn.mean(-1, keepdims=True)
    std = np.sqrt(((xn - mean) ** 2).sum(-1, keepdims=True) / (32 - 1))      # unbiased
    ref = g.numpy() * (xn - mean) / (std + 1e-6) + b.numpy()
    np.testing.assert_allclose(y.numpy(), ref, rtol=1e-12, atol=1e-12)
    # a biased estimator or eps inside the sqrt must NOT pass
    bad = g.numpy() * (xn - mean) / (np.sqrt(((xn - mean) ** 2).mean(-1, keepdims=True)) + 1e-6) + b.numpy()
    assert np.abs(bad - ref).max() > 1e-3


@pytest.mark.parametrize("mask", ["none", "causal", "key_padding"])
def test_attention_matches_sdpa(mask):
    torch.manual_seed(1)
    cfg = ol.TransformerCfg(hidden=64, heads=4, ffn=128, mask=mask)
    p = ol.init_params(cfg, 3, dtype=torch.float64, std=0.3)
    for k in p:
        if k.endswith("bias"):
            p[k] = torch.randn_like(p[k]) * 0.1
    b, s = 3, 16
    x = torch.randn(b, s, 64, dtype=torch.float64)
    lens = torch.tensor([16, 5, 9]) if mask == "key_padding" else None
    got = ol.attention(x, p, cfg, lens)
    lin = lambda i, t: F.linear(t, p[f"self_attn.linears.{i}.weight"], p[f"self_attn.linears.{i}.bias"])
    q, k, v = [lin(i, x).view(b, s, 4, 16).transpose(1, 2) for i in range(3)]
    if mask == "none":
        ctx = F.scaled_dot_product_attention(q, k, v)
    elif mask == "causal":
        ctx = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    else:
        m = (torch.arange(s).view(1, 1, 1, s) < lens.view(b, 1, 1, 1))
        ctx = F.scaled_dot_product_attention(q, k, v, attn_mask=m)
    ref = lin(3, ctx.transpose(1, 2).reshape(b, s, 64))
    torch.testing.assert_close(got, ref, rtol=1e-10, atol=1e-10)


def test_layer_matches_torch_encoder_layer():
    """Pre-LN, ReLU, standard LayerNorm, no mask == nn.TransformerEncoderLayer(norm_first=True)."""
    torch.manual_seed(2)
    h, a, f = 48, 4, 96
    cfg = ol.TransformerCfg(hidden=h, heads=a, ffn=f, activation="relu", ln="standard", mask="none")
    p = ol.init_params(cfg, 5, dtype=torch.float64, std=0.2)
    for k in p:
        if k.endswith("bias") or k.endswith("b_2"):
            p[k] = torch.randn_like(p[k]) * 0.1
        if k.endswith("a_2"):
            p[k] = 1 + 0.1 * torch.randn_like(p[k])
    ref = torch.nn.TransformerEncoderLayer(h, a, f, dropout=0.0, activation="relu", batch_first=True,
                                           norm_first=True, dtype=torch.float64)
    with torch.no_grad():
        ref.self_attn.in_proj_weight.copy_(torch.cat([p[f"self_attn.linears.{i}.weight"] for i in range(3)]))
        ref.self_attn.in_proj_bias.copy_(torch.cat([p[f"self_attn.linears.{i}.bias"] for i in range(3)]))
        ref.self_attn.out_proj.weight.copy_(p["self_attn.linears.3.weight"])
        ref.self_attn.out_proj.bias.copy_(p["self_attn.linears.3.bias"])
        ref.linear1.weight.copy_(p["feed_forward.w_1.weight"]); ref.linear1.bias.copy_(p["feed_forward.w_1.bias"])
        ref.linear2.weight.copy_(p["feed_forward.w_2.weight"]); ref.linear2.bias.copy_(p["feed_forward.w_2.bias"])
        ref.norm1.weight.copy_(p["sublayer.0.norm.a_2"]); ref.norm1.bias.copy_(p["sublayer.0.norm.b_2"])
        ref.norm2.weight.copy_(p["sublayer.1.norm.a_2"]); ref.norm2.bias.copy_(p["sublayer.1.norm.b_2"])
    x = torch.randn(2, 10, h, dtype=torch.float64)
    torch.testing.assert_close(ol.transformer_layer(x, p, cfg), ref(x), rtol=1e-9, atol=1e-9)
    cfg_c = ol.TransformerCfg(hidden=h, heads=a, ffn=f, activation="relu", ln="standard", mask="causal")
    cm = torch.nn.Transformer.generate_square_subsequent_mask(10, dtype=torch.float64)
    torch.testing.assert_close(ol.transformer_layer(x, p, cfg_c), ref(x, src_mask=cm, is_causal=True), rtol=1e-9, atol=1e-9)


@pytest.mark.parametrize("mistake", [None, "memory_from_stream", "unnormalised_queries", "memory_normalised", "wrong_sign"])
def test_decoder_layer_against_library_attention(mistake):
    """``oracle.layers.decoder_layer`` (gpt2.py:20-34) against a composition of library routines: both attentions by
    ``nn.MultiheadAttention`` (self: query = key = value = the normalised stream; memory: query = the normalised
    stream, key = value = sqrt(1 - x) of the layer's INPUT, un-normalised), LayerNorm by the closed form, the
    feed-forward by ``F.linear``; output and every gradient in fp64.  Four plausible mistakes in the composition
    (memory taken from the running stream instead of the layer input, queries not normalised, memory normalised,
    sqrt(1 + x)) each break the agreement."""
    torch.manual_seed(6)
    h, a, f, b, s = 32, 4, 64, 2, 9
    cfg = ol.TransformerCfg(hidden=h, heads=a, ffn=f, decoder=True)
    p = {k: (v.double() + 0.1 * torch.randn(v.shape, dtype=torch.float64)).requires_grad_(True)
         for k, v in ol.init_params(cfg, 3, std=0.3).items()}
    assert list(p) == list(ol.DECODER_PARAM_ORDER) and len(p) == 26
    x = (0.9 * torch.rand(b, s, h, dtype=torch.float64)).requires_grad_(True)
    dy = torch.randn(b, s, h, dtype=torch.float64)
    out = ol.decoder_layer(x, p, cfg)
    grads = torch.autograd.grad(out, [x] + list(p.values()), dy)

    def mha(prefix, q_in, kv_in):
        m = torch.nn.MultiheadAttention(h, a, batch_first=True, dtype=torch.float64)
        with torch.no_grad():
            m.in_proj_weight.copy_(torch.cat([p[f"{prefix}.linears.{i}.weight"] for i in range(3)]))
            m.in_proj_bias.copy_(torch.cat([p[f"{prefix}.linears.{i}.bias"] for i in range(3)]))
            m.out_proj.weight.copy_(p[f"{prefix}.linears.3.weight"])
            m.out_proj.bias.copy_(p[f"{prefix}.linears.3.bias"])
        return m, m(q_in, kv_in, kv_in, need_weights=False)[0]
    ln = lambda t, i: p[f"sublayer.{i}.norm.a_2"] * (t - t.mean(-1, keepdim=True)) / (t.std(-1, keepdim=True) + 1e-6) + p[f"sublayer.{i}.norm.b_2"]
    x2 = x.detach().clone().requires_grad_(True)
    mem = torch.sqrt(1 + x2) if mistake == "wrong_sign" else torch.sqrt(1 - x2)
    m0, y0 = mha("self_attn", ln(x2, 0), ln(x2, 0))
    x_1 = x2 + y0
    if mistake == "memory_from_stream":
        mem = torch.sqrt(1 - x_1.clamp(max=0.99))
    if mistake == "memory_normalised":
        mem = ln(mem, 1)
    m1, y1 = mha("src_attn", x_1 if mistake == "unnormalised_queries" else ln(x_1, 1), mem)
    x_2 = x_1 + y1
    ref = x_2 + F.linear(torch.relu(F.linear(ln(x_2, 2), p["feed_forward.w_1.weight"], p["feed_forward.w_1.bias"])),
                         p["feed_forward.w_2.weight"], p["feed_forward.w_2.bias"])
    ok = bool(torch.allclose(out, ref, rtol=1e-9, atol=1e-10))
    assert ok == (mistake is None)
    if mistake is None:
        gx, = torch.autograd.grad(ref, [x2], dy, retain_graph=True)
        assert torch.allclose(grads[0], gx, rtol=1e-8, atol=1e-10)
        # parameter gradients: the library modules hold copies, so compare through them
        ref.backward(dy)
        names = list(p)
        for prefix, mod in (("self_attn", m0), ("src_attn", m1)):
            gw = torch.cat([grads[1 + names.index(f"{prefix}.linears.{i}.weight")] for i in range(3)])
            assert torch.allclose(gw, mod.in_proj_weight.grad, rtol=1e-8, atol=1e-10)
            assert torch.allclose(grads[1 + names.index(f"{prefix}.linears.3.weight")], mod.out_proj.weight.grad, rtol=1e-8, atol=1e-10)


def test_script_tail_equals_the_module_form():
    """final LayerNorm + sum over the hidden dimension against the stand-in of the reference's LayerNorm module
    followed by the script's lambda, values and gradients."""
    from tests.reference_shapes import RefLayerNorm
    torch.manual_seed(5)
    norm = RefLayerNorm(24).double()
    with torch.no_grad():
        norm.a_2.add_(0.2 * torch.randn(24, dtype=torch.float64))
        norm.b_2.add_(0.2 * torch.randn(24, dtype=torch.float64))
    x = torch.randn(2, 7, 24, dtype=torch.float64, requires_grad=True)
    p = {"a_2": norm.a_2.detach().clone().requires_grad_(True), "b_2": norm.b_2.detach().clone().requires_grad_(True)}
    y = ol.script_tail(x, p)
    ref = (lambda t: t.sum(-1))(norm(x))
    assert y.shape == (2, 7)
    torch.testing.assert_close(y, ref, rtol=1e-12, atol=1e-12)
    w = torch.randn(2, 7, dtype=torch.float64)
    gx, ga = torch.autograd.grad((y * w).sum(), [x, p["a_2"]])
    rx, ra = torch.autograd.grad((ref * w).sum(), [x, norm.a_2])
    torch.testing.assert_close(gx, rx, rtol=1e-10, atol=1e-12)
    torch.testing.assert_close(ga, ra, rtol=1e-10, atol=1e-12)
    # with unit gain and zero shift the normalised row sums to zero: the tail's output is 0 whatever x
    unit = {"a_2": torch.ones(24, dtype=torch.float64), "b_2": torch.zeros(24, dtype=torch.float64)}
    assert float(ol.script_tail(x.detach(), unit).abs().max()) < 1e-12


def test_gelu_tanh_formula():
    x = torch.linspace(-4, 4, 101, dtype=torch.float64)
    ref = 0.5 * x * (1 + torch.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))
    torch.testing.assert_close(ol.activation(x, "gelu_tanh"), ref, rtol=1e-12, atol=1e-12)


def test_param_count_matches_reference_known_answer():
    # 12 596 224 parameters per layer at hidden 1024, ffn 4096 (tests/unit/test_partition.py:161)
    cfg = ol.TransformerCfg(hidden=1024, heads=16, ffn=4096)
    assert sum(math.prod(s) for s in ol.param_shapes(cfg).values()) == 12596224


def test_bottleneck_identity_shapes_and_relu():
    cfg = ol.BottleneckCfg(in_channels=64, mid_channels=16)
    p = ol.init_bottleneck_params(cfg, 1)
    x = torch.randn(4, 64, 6, 6)
    y = ol.bottleneck(x, p, cfg)
    assert y.shape == x.shape and (y >= 0).all()
    # zero last BN gain => residual branch vanishes => relu(x)
    p["residual_function.7.weight"].zero_()
    torch.testing.assert_close(ol.bottleneck(x, p, cfg), F.relu(x))


def _module_bottleneck(cfg):
    """The block as torch.nn modules in the arrangement of the reference's ``BottleNeck``
    (resnet.py:53-72): Sequential(conv1x1, BN, ReLU, conv3x3(stride, pad 1), BN, ReLU, conv1x1, BN),
    a shortcut Sequential (empty, or conv1x1(stride) + BN), ReLU of the sum; all convolutions bias-free."""
    nn = torch.nn
    ci, cm, co = cfg.in_channels, cfg.mid_channels, cfg.out_channels

    class Block(nn.Module):
        def __init__(self):
            super().__init__()
            self.residual_function = nn.Sequential(
                nn.Conv2d(ci, cm, 1, bias=False), nn.BatchNorm2d(cm, eps=cfg.bn_eps), nn.ReLU(),
                nn.Conv2d(cm, cm, 3, stride=cfg.stride, padding=1, bias=False), nn.BatchNorm2d(cm, eps=cfg.bn_eps), nn.ReLU(),
                nn.Conv2d(cm, co, 1, bias=False), nn.BatchNorm2d(co, eps=cfg.bn_eps))
            self.shortcut = nn.Sequential()
            if cfg.stride != 1 or ci != co:
                self.shortcut = nn.Sequential(nn.Conv2d(ci, co, 1, stride=cfg.stride, bias=False), nn.BatchNorm2d(co, eps=cfg.bn_eps))

        def forward(self, x):
            return torch.relu(self.residual_function(x) + self.shortcut(x))
    return Block().double().train()


def _bottleneck_case(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    p = ol.init_bottleneck_params(cfg, seed, dtype=torch.float64)
    for k in p:     # BN gains and shifts away from 1 / 0, so that swapping two of them shows
        if p[k].dim() == 1:
            p[k] = (1.0 if k.endswith("weight") else 0.0) + 0.3 * torch.randn(p[k].shape, generator=g, dtype=torch.float64)
    p = {k: v.requires_grad_(True) for k, v in p.items()}
    x = torch.randn(3, cfg.in_channels, 6, 6, generator=g, dtype=torch.float64, requires_grad=True)
    return p, x


def _compare_with_modules(fn, cfg, seed=4):
    """Forward and every gradient of ``fn(x, p, cfg)`` against the nn.Module block with the same weights."""
    p, x = _bottleneck_case(cfg, seed)
    ref = _module_bottleneck(cfg)
    # the oracle's parameter names are the module's: a strict load (running statistics aside) must succeed
    missing, unexpected = ref.load_state_dict({k: v.detach() for k, v in p.items()}, strict=False)
    assert not unexpected and all("running_" in k or "num_batches" in k for k in missing)
    xr = x.detach().clone().requires_grad_(True)
    y, yr = fn(x, p, cfg), ref(xr)
    dy = torch.randn(yr.shape, generator=torch.Generator().manual_seed(seed + 1), dtype=torch.float64)
    y.backward(dy)
    yr.backward(dy)
    torch.testing.assert_close(y, yr, rtol=1e-10, atol=1e-10)
    torch.testing.assert_close(x.grad, xr.grad, rtol=1e-9, atol=1e-10)
    for k, v in ref.named_parameters():
        torch.testing.assert_close(p[k].grad, v.grad, rtol=1e-9, atol=1e-10, msg=k)


@pytest.mark.parametrize("ci,cm,stride", [(64, 16, 1), (32, 16, 1), (64, 16, 2), (48, 8, 2)],
                         ids=["identity", "projection", "strided", "strided-projection"])
def test_bottleneck_equals_the_module_composition(ci, cm, stride):
    """oracle.layers.bottleneck against Conv2d / BatchNorm2d (training mode) / ReLU modules arranged as the
    reference arranges them (resnet.py:53-75), same weights, fp64: outputs, input gradient and all parameter
    gradients."""
    _compare_with_modules(ol.bottleneck, ol.BottleneckCfg(in_channels=ci, mid_channels=cm, stride=stride), seed=ci + stride)


@pytest.mark.parametrize("mistake", ["dropped-relu", "swapped-bn", "no-padding-shift", "shortcut-before-relu"])
def test_bottleneck_pin_catches_plausible_mistakes(mistake):
    """Negative controls: each of these variants of the oracle must fail the comparison above."""
    def wrong(x, p, cfg):
        bn = lambda t, i: F.batch_norm(t, None, None, p[f"residual_function.{i}.weight"], p[f"residual_function.{i}.bias"],
                                       training=True, eps=cfg.bn_eps)
        a, b = (4, 1) if mistake == "swapped-bn" else (1, 4)
        y = F.relu(bn(F.conv2d(x, p["residual_function.0.weight"]), a))
        w3 = p["residual_function.3.weight"]
        if mistake == "no-padding-shift":
            w3 = w3.flip(-1)            # a mirrored filter: what a wrong tap order gives
        y = bn(F.conv2d(y, w3, padding=1), b)
        if mistake != "dropped-relu":
            y = F.relu(y)
        y = bn(F.conv2d(y, p["residual_function.6.weight"]), 7)
        return F.relu(y) + x if mistake == "shortcut-before-relu" else F.relu(y + x)
    with pytest.raises(AssertionError):
        _compare_with_modules(wrong, ol.BottleneckCfg(in_channels=64, mid_channels=16))


def test_relu_decisions_handed_in_reproduce_the_plain_run():
    """With the decisions an exact run makes itself (x > 0) the masked variants are the plain functions, bit for
    bit, outputs and gradients; with one decision flipped they are not."""
    cfg = ol.BottleneckCfg(in_channels=64, mid_channels=16)
    p, x = _bottleneck_case(cfg, 9)
    y = ol.bottleneck(x, p, cfg)
    y.sum().backward()
    gx = x.grad.clone()
    bn = lambda t, i: F.batch_norm(t, None, None, p[f"residual_function.{i}.weight"], p[f"residual_function.{i}.bias"], training=True, eps=cfg.bn_eps)
    with torch.no_grad():
        u1 = bn(F.conv2d(x, p["residual_function.0.weight"]), 1)
        u2 = bn(F.conv2d(F.relu(u1), p["residual_function.3.weight"], padding=1), 4)
        u3 = bn(F.conv2d(F.relu(u2), p["residual_function.6.weight"]), 7) + x
    masks = (u1 > 0, u2 > 0, u3 > 0)
    x.grad = None
    ym = ol.bottleneck(x, p, cfg, masks)
    ym.sum().backward()
    assert torch.equal(ym, y) and torch.equal(x.grad, gx)
    flipped = (masks[0].clone(), masks[1], masks[2])
    flipped[0][0, 0, 0, 0] = ~flipped[0][0, 0, 0, 0]
    assert not torch.equal(ol.bottleneck(x, p, cfg, flipped), y)
    # transformer feed-forward
    tcfg = ol.TransformerCfg(hidden=32, heads=4, ffn=64)
    tp = {k: v.double() for k, v in ol.init_params(tcfg, 3).items()}
    t = torch.randn(2, 5, 32, dtype=torch.float64)
    u = F.linear(t, tp["feed_forward.w_1.weight"], tp["feed_forward.w_1.bias"])
    assert torch.equal(ol.feed_forward(t, tp, tcfg, u > 0), ol.feed_forward(t, tp, tcfg))


@pytest.mark.parametrize("adam_w,wd", [(True, 0.0), (True, 0.01), (False, 0.01)])
def test_adam_matches_torch(adam_w, wd):
    torch.manual_seed(3)
    n = 1031
    p0 = torch.randn(n)
    p_t = p0.clone().requires_grad_(True)
    opt = (torch.optim.AdamW if adam_w else torch.optim.Adam)([p_t], lr=1e-3, betas=(0.9, 0.999), eps=1e-8, weight_decay=wd)
    p, m, v = p0.numpy().copy(), np.zeros(n, np.float32), np.zeros(n, np.float32)
    for step in range(1, 11):
        g = torch.randn(n)
        p_t.grad = g.clone()
        opt.step()
        oadam.adam_step(p, g.numpy(), m, v, step, weight_decay=wd, adam_w_mode=adam_w)
        np.testing.assert_allclose(p, p_t.detach().numpy(), rtol=2e-6, atol=2e-7)


@pytest.mark.parametrize("max_norm", [0.5, 1e6])
def test_clip_grad_norm_matches_torch(max_norm):
    """The restated global-norm clipping against torch.nn.utils.clip_grad_norm_ (the routine the reference's
    clip_grad_norm_ is adapted from: same coefficient max_norm / (norm + 1e-6), applied only below 1), on tensors of
    different sizes; a bound far above the norm leaves the gradients untouched bit for bit."""
    torch.manual_seed(4)
    params = [torch.nn.Parameter(torch.zeros(n)) for n in (7, 1024, 33)]
    for prm in params:
        prm.grad = torch.randn_like(prm) * 3
    grads = [prm.grad.numpy().copy() for prm in params]
    before = [g.copy() for g in grads]
    norm_t = float(torch.nn.utils.clip_grad_norm_(params, max_norm))
    norm, coef = oadam.clip_grad_norm(grads, max_norm)
    assert abs(norm - norm_t) < 1e-5 * norm_t
    want = (sum(float((b.astype(np.float64) ** 2).sum()) for b in before)) ** 0.5      # the closed form
    assert abs(norm - want) < 1e-12 * want and abs(coef - max_norm / (want + 1e-6)) < 1e-12
    for g, prm, b in zip(grads, params, before):
        np.testing.assert_allclose(g, prm.grad.numpy(), rtol=1e-6, atol=0)
        if max_norm > 1e5:
            assert np.array_equal(g, b)
        else:
            assert abs(float(np.abs(g).max()) / float(np.abs(b).max()) - coef) < 1e-6


def test_adam_first_step_closed_form():
    # step 1 with zero moments: update = g / (|g| + eps*sqrt(1-b2)) ~ sign(g): p1 = p0 - lr*sign(g)
    p = np.array([1.0, -2.0, 3.0], np.float32)
    g = np.array([0.5, -0.25, 4.0], np.float32)
    m, v = np.zeros(3, np.float32), np.zeros(3, np.float32)
    oadam.adam_step(p, g, m, v, 1, lr=0.1)
    np.testing.assert_allclose(p, [0.9, -1.9, 2.9], rtol=1e-5)


def test_batch_statistics_from_strips_equal_the_direct_ones():
    """The strip restatement of BatchNorm's batch statistics (what the convolution epilogues and the finish
    kernel compute) is an identity: checked against torch's mean / var on data with a mean far from zero,
    a ragged last strip, and a single-strip tensor."""
    g = torch.Generator().manual_seed(5)
    for rows, cols, shift in ((6272, 24, 0.0), (300, 8, 50.0), (20, 16, -3.0), (33, 8, 1e3)):
        y = torch.randn(rows, cols, generator=g, dtype=torch.float64) * 0.7 + shift
        mean, var = ol.batch_stats_from_strips(ol.strip_triples(y), rows)
        torch.testing.assert_close(mean, y.mean(0), rtol=1e-12, atol=1e-12)
        torch.testing.assert_close(var, y.var(0, unbiased=False), rtol=1e-9, atol=1e-12)
    # one row per strip degenerates to the textbook two-pass formula
    y = torch.randn(7, 4, generator=g, dtype=torch.float64)
    mean, var = ol.batch_stats_from_strips(ol.strip_triples(y, strip=1), 7, strip=1)
    torch.testing.assert_close(var, ((y - y.mean(0)) ** 2).mean(0))
