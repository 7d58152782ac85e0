"""Layer mathematics of the reference models on torch CPU ops (TEST ORACLE).

Follows DeepSpeedExamples/pipeline_parallelism/transformer.py of the reference:
  layer_norm          transformer.py:77-88   (LayerNorm: unbiased std, eps outside sqrt)
  attention           transformer.py:106-146 (MultiHeadedAttention, masked_fill(mask==0,-1e9))
  feed_forward        transformer.py:149-158 (PositionwiseFeedForward)
  transformer_layer   transformer.py:91-103,161-172 (SublayerConnection + EncoderLayer, pre-LN)
  decoder_layer       gpt2.py:20-34          (DecoderLayerSimple: self-attention, attention over
                      m = sqrt(1 - x) of the layer's input, feed-forward; three pre-LN residual sublayers)
  script_tail         transformer.py:181,250 (final LayerNorm, then sum over the hidden dimension)
  bottleneck          resnet.py:49-75        (BottleNeck, bias-free convs, train-mode BN)
  batch_stats_from_strips  resnet.py:56,59,62 (nn.BatchNorm2d batch statistics, restated over
                      32-row strips as the HIP path computes them; pinned against torch's
                      mean / var in tests/test_oracle_layers.py)
Dropout is fixed to 0 (the reference's own parity test disables it,
tests/unit/test_pipe.py:144-145).  Switches beyond the reference's setting
(`relu`, `annotated`, no mask) exist because the benchmark configurations ask
for causal / key-padding masks, tanh-GELU and the standard LayerNorm.
"""
import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F

PARAM_ORDER = (
    "sublayer.0.norm.a_2", "sublayer.0.norm.b_2",
    "self_attn.linears.0.weight", "self_attn.linears.0.bias",
    "self_attn.linears.1.weight", "self_attn.linears.1.bias",
    "self_attn.linears.2.weight", "self_attn.linears.2.bias",
    "self_attn.linears.3.weight", "self_attn.linears.3.bias",
    "sublayer.1.norm.a_2", "sublayer.1.norm.b_2",
    "feed_forward.w_1.weight", "feed_forward.w_1.bias",
    "feed_forward.w_2.weight", "feed_forward.w_2.bias",
)


@dataclass(frozen=True)
class TransformerCfg:
    hidden: int
    heads: int
    ffn: int
    activation: str = "relu"      # relu | gelu_tanh
    ln: str = "annotated"         # annotated (reference) | standard
    mask: str = "none"            # none | causal | key_padding
    ln_eps: float = None
    dropout: float = 0.0          # the reference scripts run 0.1 (transformer.py:196); masks are handed in explicitly
    decoder: bool = False         # the GPT-2 script's DecoderLayerSimple (gpt2.py:20-34) instead of EncoderLayer

    @property
    def eps(self):
        if self.ln_eps is not None:
            return self.ln_eps
        return 1e-6 if self.ln == "annotated" else 1e-5


# registration order of DecoderLayerSimple's parameters (self_attn, src_attn, feed_forward, sublayer: gpt2.py:22-27)
DECODER_PARAM_ORDER = tuple(
    [f"self_attn.linears.{i}.{k}" for i in range(4) for k in ("weight", "bias")] +
    [f"src_attn.linears.{i}.{k}" for i in range(4) for k in ("weight", "bias")] +
    ["feed_forward.w_1.weight", "feed_forward.w_1.bias", "feed_forward.w_2.weight", "feed_forward.w_2.bias"] +
    [f"sublayer.{i}.norm.{k}" for i in range(3) for k in ("a_2", "b_2")])


def param_shapes(cfg):
    h, f = cfg.hidden, cfg.ffn
    if cfg.decoder:
        shape = lambda n: (f, h) if n == "feed_forward.w_1.weight" else (h, f) if n == "feed_forward.w_2.weight" else \
            (f,) if n == "feed_forward.w_1.bias" else (h, h) if n.endswith("weight") else (h,)
        return {n: shape(n) for n in DECODER_PARAM_ORDER}
    return {
        "sublayer.0.norm.a_2": (h,), "sublayer.0.norm.b_2": (h,),
        "self_attn.linears.0.weight": (h, h), "self_attn.linears.0.bias": (h,),
        "self_attn.linears.1.weight": (h, h), "self_attn.linears.1.bias": (h,),
        "self_attn.linears.2.weight": (h, h), "self_attn.linears.2.bias": (h,),
        "self_attn.linears.3.weight": (h, h), "self_attn.linears.3.bias": (h,),
        "sublayer.1.norm.a_2": (h,), "sublayer.1.norm.b_2": (h,),
        "feed_forward.w_1.weight": (f, h), "feed_forward.w_1.bias": (f,),
        "feed_forward.w_2.weight": (h, f), "feed_forward.w_2.bias": (h,),
    }


def init_params(cfg, seed, dtype=torch.float32, std=0.02):
    """Weights N(0, std) from a per-tensor seeded generator, biases 0, LN gain 1."""
    out = {}
    for i, (name, shape) in enumerate(param_shapes(cfg).items()):
        if name.endswith("a_2"):
            t = torch.ones(shape, dtype=dtype)
        elif name.endswith("weight"):
            g = torch.Generator().manual_seed(seed * 1000 + i)
            t = (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)
        else:
            t = torch.zeros(shape, dtype=dtype)
        out[name] = t
    return out


def layer_norm(x, gain, shift, kind, eps):
    if kind == "annotated":
        mean = x.mean(-1, keepdim=True)
        std = x.std(-1, keepdim=True)            # unbiased (n-1)
        return gain * (x - mean) / (std + eps) + shift
    return F.layer_norm(x, x.shape[-1:], gain, shift, eps)


# Set to a list by a test that hands a low-precision run's ReLU decisions to the oracle: every ReLU evaluated with
# such decisions appends (elements, elements whose decision differs from the oracle's own x > 0, the largest |x|
# among those, the largest |x| of the tensor).  Decisions may differ only where x is within rounding of zero.
RELU_AUDIT = None


def activation(x, kind, mask=None):
    """``mask`` (relu only): use this 0/1 tensor as the ReLU's decision instead of ``x > 0``.  A low-precision
    run decides ``x > 0`` on its own rounded ``x``; for the few pre-activations closer to zero than the
    rounding error the decision differs from the exact one and the derivative jumps.  Feeding the run's own
    decisions makes the comparison one of arithmetic, not of tie-breaking at the kink."""
    if kind == "relu":
        if mask is None:
            return F.relu(x)
        if RELU_AUDIT is not None:
            # what the handed-in decisions differ in from the oracle's own ``x > 0``, for the caller to bound
            xd = x.detach()
            differ = (xd > 0) != mask.to(torch.bool).view_as(xd)
            worst = float(xd.abs()[differ].max()) if bool(differ.any()) else 0.0
            RELU_AUDIT.append((xd.numel(), int(differ.sum()), worst, float(xd.abs().max())))
        return x * mask.to(x.dtype)
    if kind == "gelu_tanh":
        return F.gelu(x, approximate="tanh")
    raise ValueError(kind)


def build_mask(cfg, batch, seq, key_lens=None):
    """Boolean [b,1,s,s] / [b,1,1,s] mask, True = keep (reference: mask == 0 is filled)."""
    if cfg.mask == "none":
        return None
    if cfg.mask == "causal":
        return torch.tril(torch.ones(seq, seq, dtype=torch.bool)).view(1, 1, seq, seq)
    if cfg.mask == "key_padding":
        ar = torch.arange(seq).view(1, 1, 1, seq)
        return ar < key_lens.view(batch, 1, 1, 1)
    raise ValueError(cfg.mask)


def drop(x, mask, p_drop):
    """nn.Dropout in training mode with a given 0/1 mask: kept elements scaled by 1 / (1 - p)."""
    if mask is None:
        return x
    return x * mask.to(x.dtype).view_as(x) / (1.0 - p_drop)


def attention(x, p, cfg, key_lens=None, prob_mask=None, memory=None, prefix="self_attn"):
    """``memory``: keys and values are projected from it instead of from ``x`` (MultiHeadedAttention(query, key, value)
    with key = value = memory, gpt2.py:33), and no mask applies."""
    b, s, h = x.shape
    a, d = cfg.heads, cfg.hidden // cfg.heads
    lin = lambda i, t: F.linear(t, p[f"{prefix}.linears.{i}.weight"], p[f"{prefix}.linears.{i}.bias"])
    kv_in = x if memory is None else memory
    q, k, v = [lin(i, t).view(b, s, a, d).transpose(1, 2) for i, t in ((0, x), (1, kv_in), (2, kv_in))]
    scores = torch.matmul(q, k.transpose(-2, -1)) / math.sqrt(d)
    mask = build_mask(cfg, b, s, key_lens) if memory is None else None
    if mask is not None:
        scores = scores.masked_fill(~mask, -1e9)
    prob = drop(F.softmax(scores, dim=-1), prob_mask, cfg.dropout)          # transformer.py:125-126
    ctx = torch.matmul(prob, v).transpose(1, 2).contiguous().view(b, s, h)
    return lin(3, ctx)


def feed_forward(x, p, cfg, relu_mask=None, hidden_mask=None):
    u = F.linear(x, p["feed_forward.w_1.weight"], p["feed_forward.w_1.bias"])
    a = drop(activation(u, cfg.activation, relu_mask), hidden_mask, cfg.dropout)    # transformer.py:158
    return F.linear(a, p["feed_forward.w_2.weight"], p["feed_forward.w_2.bias"])


def decoder_layer(x, p, cfg, key_lens=None, relu_mask=None, drop_masks=None):
    """DecoderLayerSimple.forward (gpt2.py:29-34).  Dropout sites: 0 self-attention probabilities, 1 first sublayer,
    4 memory-attention probabilities, 5 second sublayer, 2 feed-forward hidden, 3 last sublayer."""
    dm = drop_masks or {}
    norm = lambda t, i: layer_norm(t, p[f"sublayer.{i}.norm.a_2"], p[f"sublayer.{i}.norm.b_2"], cfg.ln, cfg.eps)
    m = torch.sqrt(1 - x)                                                                              # gpt2.py:31
    x = x + drop(attention(norm(x, 0), p, cfg, key_lens, dm.get(0)), dm.get(1), cfg.dropout)          # :32
    x = x + drop(attention(norm(x, 1), p, cfg, None, dm.get(4), memory=m, prefix="src_attn"), dm.get(5), cfg.dropout)   # :33
    return x + drop(feed_forward(norm(x, 2), p, cfg, relu_mask, dm.get(2)), dm.get(3), cfg.dropout)  # :34


def transformer_layer(x, p, cfg, key_lens=None, relu_mask=None, drop_masks=None):
    """``drop_masks``: {site: 0/1 tensor} for the layer's four dropout sites (oracle.dropout.SITE_*): attention
    probabilities [b, heads, s, s], sublayer outputs [b, s, h], feed-forward hidden [b, s, ffn]."""
    if cfg.decoder:
        return decoder_layer(x, p, cfg, key_lens, relu_mask, drop_masks)
    dm = drop_masks or {}
    n1 = layer_norm(x, p["sublayer.0.norm.a_2"], p["sublayer.0.norm.b_2"], cfg.ln, cfg.eps)
    x = x + drop(attention(n1, p, cfg, key_lens, dm.get(0)), dm.get(1), cfg.dropout)      # transformer.py:103
    n2 = layer_norm(x, p["sublayer.1.norm.a_2"], p["sublayer.1.norm.b_2"], cfg.ln, cfg.eps)
    return x + drop(feed_forward(n2, p, cfg, relu_mask, dm.get(2)), dm.get(3), cfg.dropout)


def layer_drop_masks(cfg, base_seed, step, micro_batch, layer_idx, batch, seq):
    """The four masks of one layer forward under this build's decision function (oracle.dropout)."""
    from . import dropout as od
    shapes = {od.SITE_ATTENTION: (batch, cfg.heads, seq, seq), od.SITE_SUBLAYER0: (batch, seq, cfg.hidden),
              od.SITE_FFN: (batch, seq, cfg.ffn), od.SITE_SUBLAYER1: (batch, seq, cfg.hidden)}
    if cfg.decoder:
        shapes.update({4: (batch, cfg.heads, seq, seq), 5: (batch, seq, cfg.hidden)})
    return {site: torch.from_numpy(od.mask(cfg.dropout, od.key(base_seed, step, micro_batch, layer_idx, site), shape))
            for site, shape in shapes.items()}


def script_tail(x, p, kind="annotated", eps=1e-6):
    """The two layers that end the reference's transformer script (transformer.py:250): the encoder's final
    LayerNorm (:181, parameters a_2 / b_2) and ``lambda x: x.sum(-1)``; [b, s, h] -> [b, s], to be compared with
    [b, s] labels by ``nn.MSELoss()`` (:205-219, :264)."""
    return layer_norm(x, p["a_2"], p["b_2"], kind, eps).sum(-1)


# ---------------------------------------------------------------- ResNet bottleneck

@dataclass(frozen=True)
class BottleneckCfg:
    in_channels: int = 1024
    mid_channels: int = 256
    stride: int = 1
    bn_eps: float = 1e-5

    @property
    def out_channels(self):
        return 4 * self.mid_channels


    @property
    def projection(self):
        """The shortcut is conv1x1(stride) + BN instead of the identity (resnet.py:68-72)."""
        return self.stride != 1 or self.in_channels != self.out_channels


def bottleneck_param_shapes(cfg):
    ci, cm, co = cfg.in_channels, cfg.mid_channels, cfg.out_channels
    shapes = {
        "residual_function.0.weight": (cm, ci, 1, 1),
        "residual_function.1.weight": (cm,), "residual_function.1.bias": (cm,),
        "residual_function.3.weight": (cm, cm, 3, 3),
        "residual_function.4.weight": (cm,), "residual_function.4.bias": (cm,),
        "residual_function.6.weight": (co, cm, 1, 1),
        "residual_function.7.weight": (co,), "residual_function.7.bias": (co,),
    }
    if cfg.projection:
        shapes.update({"shortcut.0.weight": (co, ci, 1, 1), "shortcut.1.weight": (co,), "shortcut.1.bias": (co,)})
    return shapes


def init_bottleneck_params(cfg, seed, dtype=torch.float32):
    """He-normal conv weights (std = sqrt(2/fan_in)), BN gamma 1 / beta 0."""
    out = {}
    for i, (name, shape) in enumerate(bottleneck_param_shapes(cfg).items()):
        if len(shape) == 4:
            fan_in = shape[1] * shape[2] * shape[3]
            g = torch.Generator().manual_seed(seed * 1000 + i)
            t = torch.randn(shape, generator=g, dtype=torch.float32) * math.sqrt(2.0 / fan_in)
        elif name.endswith("weight"):
            t = torch.ones(shape)
        else:
            t = torch.zeros(shape)
        out[name] = t.to(dtype)
    return out


def bottleneck(x, p, cfg, relu_masks=None):
    """x is NCHW here (torch's convention).  Shortcut: the identity when stride is 1 and
    Cin == 4*Cmid, else conv1x1(stride) + BN (resnet.py:66-72).  ``relu_masks``: the decisions of
    the block's three ReLUs, in order, to use instead of ``> 0`` (see :func:`activation`)."""
    bn = lambda t, key: F.batch_norm(t, None, None, p[f"{key}.weight"], p[f"{key}.bias"], training=True, eps=cfg.bn_eps)
    m = relu_masks if relu_masks is not None else (None, None, None)
    y = activation(bn(F.conv2d(x, p["residual_function.0.weight"]), "residual_function.1"), "relu", m[0])
    y = activation(bn(F.conv2d(y, p["residual_function.3.weight"], stride=cfg.stride, padding=1), "residual_function.4"), "relu", m[1])
    y = bn(F.conv2d(y, p["residual_function.6.weight"]), "residual_function.7")
    sc = x
    if cfg.projection:
        sc = bn(F.conv2d(x, p["shortcut.0.weight"], stride=cfg.stride), "shortcut.1")
    return activation(y + sc, "relu", m[2])


def strip_triples(y, strip=32):
    """Per strip of `strip` consecutive rows and per column: (pivot = the strip's first row,
    sum (y - pivot), sum (y - pivot)^2).  y: [rows, cols]; returns [strips, 3, cols] in float64."""
    yd = y.double()
    out = []
    for s0 in range(0, yd.shape[0], strip):
        blk = yd[s0:s0 + strip]
        d = blk - blk[0]
        out.append(torch.stack([blk[0], d.sum(0), (d * d).sum(0)]))
    return torch.stack(out)


def batch_stats_from_strips(triples, rows, strip=32):
    """Mean and biased variance over all rows from the strip triples: a strip's mean is
    pivot + S1/n and its sum of squared deviations S2 - S1^2/n; the batch mean is the
    n-weighted mean of the strip means, the batch sum of squared deviations is
    sum_s [M2_s + n_s (mean_s - mean)^2]."""
    ns = torch.tensor([min(strip, rows - i * strip) for i in range(triples.shape[0])], dtype=torch.float64)[:, None]
    piv, s1, s2 = triples[:, 0], triples[:, 1], triples[:, 2]
    mean_s = piv + s1 / ns
    m2_s = s2 - s1 * s1 / ns
    mean = (ns * mean_s).sum(0) / rows
    m2 = (m2_s + ns * (mean_s - mean) ** 2).sum(0)
    return mean, m2 / rows
