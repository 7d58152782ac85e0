"""Layers of a pipeline stage, executed by the gfx950 kernels of ``libbamboo_hip.so``.

``TransformerLayer`` computes what the reference's ``EncoderLayer`` computes
(DeepSpeedExamples/pipeline_parallelism/transformer.py:77-172: pre-LN residual blocks around
multi-head self-attention and a position-wise feed-forward), with explicit forward and
backward passes instead of autograd: every tensor the backward needs is written once, by the
kernel that produces it, into a per-micro-batch *stash* slot in HBM.  Parameter names are
the reference module's (``self_attn.linears.0.weight`` ...), so ``"{layer_idx}.{name}"`` keys
of the reference's parameter buffers (module.py:229-246) carry over.

Memory layout.  Activations are ``[rows, features]`` row-major with ``rows = batch * seq``.
Heads are never split out: Q, K and V of head ``j`` are the column slices
``[j*d, (j+1)*d)`` of the three thirds of the ``[rows, 3*hidden]`` QKV buffer, and the
batched GEMMs walk them with (batch, head) strides.  The Q/K/V projection weights are three
adjacent ``[hidden, hidden]`` blocks of one ``[3*hidden, hidden]`` allocation, so the three
``nn.Linear`` calls of the reference become a single GEMM.
"""
import math
from collections import OrderedDict

import torch

from . import hip


class StageContext:
    """Per-execution-lane state shared by the layers of a stage: shapes, dtype, the stream the
    kernels go to, backward scratch and reduction workspaces."""

    def __init__(self, batch, seq, dtype, device, stream=None):
        self.batch, self.seq, self.dtype, self.device = batch, seq, dtype, device
        self.stream = stream
        self.scratch = {}
        self.key_len = None
        self.workspace = None
        # (base seed, batch counter, micro-batch): with a layer's index and the site inside it this names a dropout
        # mask; set per forward / backward call by whoever drives the stage
        self.dropout_base = None
        self.redundant = False   # set per forward call: a redundant forward must not touch running statistics
        # set per forward call: leave out what only a backward pass reads (a redundant forward's stash is used
        # by a backward pass only after a failover); ``deferred`` tells that backward pass to produce it first
        self.defer = False
        self.deferred = False
        # optional observer of this lane's GEMM launches (``hip.gemm(..., hook=)``); set through the engine that owns
        # the context, so a probe on one engine sees and changes nothing of another
        self.gemm_hook = None
        # hand-over between two neighbouring layers of a backward pass: what the layer that receives this layer's
        # input gradient wants done to it on the way (``grad_sink``, offered by ``PipelineModule.backward``), whether
        # this layer did it (``grad_sink_used``), and whether the gradient this layer receives had it done
        # (``grad_presummed``)
        self.grad_sink = None
        self.grad_sink_used = False
        self.grad_presummed = False

    def gemm(self, *a, **kw):
        return hip.gemm(*a, hook=self.gemm_hook, **kw)

    def gemm_grouped(self, *a, **kw):
        return hip.gemm_grouped(*a, hook=self.gemm_hook, **kw)

    def conv3x3(self, *a, **kw):
        return hip.conv3x3(*a, hook=self.gemm_hook, **kw)

    def gemm_bn_bwd(self, *a, **kw):
        return hip.gemm_bn_bwd(*a, hook=self.gemm_hook, **kw)

    def conv3x3_dgrad_bn(self, *a, **kw):
        return hip.conv3x3_dgrad_bn(*a, hook=self.gemm_hook, **kw)

    @property
    def rows(self):
        return self.batch * self.seq

    def ensure_scratch(self, specs):
        for name, shape, dtype in specs:
            cur = self.scratch.get(name)
            n = math.prod(shape)
            if cur is None or cur.numel() < n or cur.dtype != dtype:
                self.scratch[name] = torch.empty(n, dtype=dtype, device=self.device)

    def ensure_workspace(self, n):
        if self.workspace is None or self.workspace.numel() < n:
            self.workspace = torch.empty(n, dtype=torch.float32, device=self.device)

    def buf(self, name, shape):
        return self.scratch[name][: math.prod(shape)].view(shape)


class TransformerLayer:
    """Pre-LN transformer layer: ``x + Attn(LN(x))`` then ``x + FFN(LN(x))``.

    activation: ``relu`` (reference) or ``gelu_tanh``; ln: ``annotated`` (reference: unbiased
    std, eps added to the std) or ``standard``; mask: ``none`` (reference scripts), ``causal``
    or ``key_padding``.

    dropout: probability of the reference's four ``nn.Dropout`` sites (attention probabilities, the two sublayer
    outputs, the feed-forward's hidden activation; transformer.py:98-103,125-126,154-158).  No mask is stored: each
    decision is a pure function of (base seed, batch counter, micro-batch, layer, site, element), evaluated inside
    the attention kernels and the GEMM epilogues, so the redundant forward of a layer, its normal forward and its
    backward pass agree bit for bit.
    """

    SITE_ATTENTION, SITE_SUBLAYER0, SITE_FFN, SITE_SUBLAYER1 = 0, 1, 2, 3

    # parameter registration order of the reference's ``EncoderLayer`` (self_attn, feed_forward, sublayer:
    # transformer.py:161-168): the order of its ``state_dict()``, hence of the layer wire format
    REFERENCE_ORDER = (
        "self_attn.linears.0.weight", "self_attn.linears.0.bias", "self_attn.linears.1.weight", "self_attn.linears.1.bias",
        "self_attn.linears.2.weight", "self_attn.linears.2.bias", "self_attn.linears.3.weight", "self_attn.linears.3.bias",
        "feed_forward.w_1.weight", "feed_forward.w_1.bias", "feed_forward.w_2.weight", "feed_forward.w_2.bias",
        "sublayer.0.norm.a_2", "sublayer.0.norm.b_2", "sublayer.1.norm.a_2", "sublayer.1.norm.b_2")

    def __init__(self, hidden, heads, ffn, activation="relu", ln="annotated", mask="none", ln_eps=None,
                 init_std=0.02, dropout=0.0):
        if hidden % heads:
            raise ValueError("hidden must be divisible by heads")
        if not 0.0 <= dropout < 1.0:
            raise ValueError("dropout must be in [0, 1)")
        self.dropout = float(dropout)
        self.layer_idx = None     # global index, set when the layer is bound to a stage's arenas
        self.hidden, self.heads, self.ffn = hidden, heads, ffn
        self.head_dim = hidden // heads
        if activation not in hip.ACT_CODES or ln not in hip.LN_CODES or mask not in hip.MASK_CODES:
            raise ValueError(f"unsupported variant activation={activation} ln={ln} mask={mask}")
        self.activation, self.ln, self.mask = activation, ln, mask
        self.eps = ln_eps if ln_eps is not None else (1e-6 if ln == "annotated" else 1e-5)
        self.init_std = init_std
        self.w = self.g = None

    # ------------------------------------------------------------------ parameters
    def param_specs(self):
        h, f = self.hidden, self.ffn
        return OrderedDict([
            ("sublayer.0.norm.a_2", (h,)), ("sublayer.0.norm.b_2", (h,)),
            ("self_attn.linears.0.weight", (h, h)), ("self_attn.linears.1.weight", (h, h)),
            ("self_attn.linears.2.weight", (h, h)),
            ("self_attn.linears.0.bias", (h,)), ("self_attn.linears.1.bias", (h,)),
            ("self_attn.linears.2.bias", (h,)),
            ("self_attn.linears.3.weight", (h, h)), ("self_attn.linears.3.bias", (h,)),
            ("sublayer.1.norm.a_2", (h,)), ("sublayer.1.norm.b_2", (h,)),
            ("feed_forward.w_1.weight", (f, h)), ("feed_forward.w_1.bias", (f,)),
            ("feed_forward.w_2.weight", (h, f)), ("feed_forward.w_2.bias", (h,)),
        ])

    def num_params(self):
        return sum(math.prod(s) for s in self.param_specs().values())

    def init_params(self, master, seed):
        """Fill fp32 master views: weights N(0, init_std) from per-tensor seeded CPU generators
        (index = position in the reference module's parameter order), biases 0, LN gain 1."""
        order = ("sublayer.0.norm.a_2", "sublayer.0.norm.b_2",
                 "self_attn.linears.0.weight", "self_attn.linears.0.bias",
                 "self_attn.linears.1.weight", "self_attn.linears.1.bias",
                 "self_attn.linears.2.weight", "self_attn.linears.2.bias",
                 "self_attn.linears.3.weight", "self_attn.linears.3.bias",
                 "sublayer.1.norm.a_2", "sublayer.1.norm.b_2",
                 "feed_forward.w_1.weight", "feed_forward.w_1.bias",
                 "feed_forward.w_2.weight", "feed_forward.w_2.bias")
        for i, name in enumerate(order):
            t = master[name]
            if name.endswith("a_2"):
                t.fill_(1.0)
            elif name.endswith("weight"):
                g = torch.Generator().manual_seed(seed * 1000 + i)
                t.copy_(torch.randn(t.shape, generator=g, dtype=torch.float32) * self.init_std)
            else:
                t.zero_()

    def bind(self, compute, grads):
        """compute / grads: name -> view (compute dtype / fp32) inside the stage's flat arenas."""
        h = self.hidden
        w, g = dict(compute), dict(grads)
        # fused QKV views over the three adjacent blocks
        for d, src in ((w, compute), (g, grads)):
            q = src["self_attn.linears.0.weight"]
            d["qkv.weight"] = torch.as_strided(q, (3 * h, h), (h, 1))
            b = src["self_attn.linears.0.bias"]
            d["qkv.bias"] = torch.as_strided(b, (3 * h,), (1,))
        self.w, self.g = w, g

    # ------------------------------------------------------------------ memory plans
    @property
    def feature_dim(self):
        return self.hidden

    @property
    def out_features(self):
        return self.hidden

    def fused_attention(self, ctx):
        """bf16 with 64- or 128-wide heads, or with an even number of 32-wide heads (the reference's GPT-2 script
        defaults to 512 / 16 = 32, gpt2.py:212-214: the kernels then take the heads in pairs), runs the fused attention
        kernels (no score matrix in HBM).  Everything else -- fp32, the correctness configuration, and bf16 with another
        head width -- materialises the probabilities like the reference does: batched head products and the masked
        softmax kernels."""
        return ctx.dtype == torch.bfloat16 and (self.head_dim in (64, 128) or (self.head_dim == 32 and self.heads % 2 == 0))

    def stash_specs(self, ctx):
        R, h, f = ctx.rows, self.hidden, self.ffn
        dt, f32 = ctx.dtype, torch.float32
        attn = ("lse", (ctx.batch, self.heads, ctx.seq), f32) if self.fused_attention(ctx) else \
            ("prob", (ctx.batch, self.heads, ctx.seq, ctx.seq), dt)
        # ReLU's derivative is read off its kept output (relu'(u) = [relu(u) > 0]); other activations keep act'
        dact = [] if self.activation == "relu" else [("dact", (R, f), dt)]
        return [
            ("n1", (R, h), dt), ("qkv", (R, 3 * h), dt), attn,
            ("ctx", (R, h), dt), ("x1", (R, h), dt), ("n2", (R, h), dt),
            *dact, ("act", (R, f), dt), ("out", (R, h), dt),
            ("mean1", (R,), f32), ("rinv1", (R,), f32), ("mean2", (R,), f32), ("rinv2", (R,), f32),
        ]

    def scratch_specs(self, ctx):
        R, h, f = ctx.rows, self.hidden, self.ffn
        dt = ctx.dtype
        attn = ("attn_delta", (ctx.batch, self.heads, ctx.seq), torch.float32) if self.fused_attention(ctx) else \
            ("d_prob", (ctx.batch, self.heads, ctx.seq, ctx.seq), dt)
        specs = [("d_ffn", (R, f), dt), ("d_h0", (R, h), dt), ("d_h1", (R, h), dt), ("d_qkv", (R, 3 * h), dt), attn]
        if self.dropout > 0:
            # the gradients behind the two sublayer dropouts: the weight gradients read them at the end of the layer
            specs += [("d_drop0", (R, h), dt), ("d_drop1", (R, h), dt)]
        return specs + self.forward_scratch_specs(ctx)

    def forward_scratch_specs(self, ctx):
        if self.dropout > 0 and not self.fused_attention(ctx):
            return [("prob_drop", (ctx.batch, self.heads, ctx.seq, ctx.seq), ctx.dtype)]   # dropped-out probabilities
        return []

    def _drop(self, ctx, site):
        """``(p, key)`` of one dropout site for the call in progress, or None."""
        if self.dropout <= 0:
            return None
        if ctx.dropout_base is None or self.layer_idx is None:
            raise hip.HipKernelError("a layer with dropout needs ctx.dropout_base = (base seed, batch counter, micro-batch) "
                                     "and its layer index")
        return self.dropout, hip.dropout_key(*ctx.dropout_base, self.layer_idx, site)

    def workspace_elems(self):
        n = max(self.hidden * 3, self.ffn)
        return max(hip.layernorm_bwd_workspace(self.hidden), hip.colsum_workspace(n))

    def flops_fwd(self, batch, seq):
        h, f = self.hidden, self.ffn
        return batch * seq * (8 * h * h + 4 * h * f) + 4 * batch * seq * seq * h

    # ------------------------------------------------------------------ attention core
    def _heads_gemm(self, ctx, layout, M, N, K, A, lda, sA, B, ldb, sB, C, ldc, sC, alpha=1.0):
        hip.gemm_batched(layout, hip.dtype_code(ctx.dtype), M, N, K, A, lda, sA, B, ldb, sB, C, ldc, sC,
                         ctx.batch, self.heads, alpha=alpha, stream=ctx.stream)

    def _attention_fwd(self, st, ctx, site=0, mask=None):
        """``st``: the entries ``qkv`` ([rows, 3h]: queries, keys, values side by side), ``ctx`` and ``lse`` / ``prob``;
        ``site``: the dropout site of the probabilities; ``mask``: the layer's own unless given."""
        h, d, s = self.hidden, self.head_dim, ctx.seq
        mask = self.mask if mask is None else mask
        drop = self._drop(ctx, site)
        if self.fused_attention(ctx):
            hip.attention_fwd(st["qkv"], st["ctx"], st["lse"], ctx.batch, self.heads, s, hip.MASK_CODES[mask],
                              ctx.key_len if mask == "key_padding" else None, stream=ctx.stream, dropout=drop)
            return
        es = st["qkv"].element_size()
        q = st["qkv"].data_ptr()
        k, v = q + h * es, q + 2 * h * es
        head_in = (s * 3 * h, d)               # (batch, head) strides inside the QKV buffer
        prob = st["prob"]
        # scores = Q K^T / sqrt(d)
        self._heads_gemm(ctx, hip.NT, s, s, d, q, 3 * h, head_in, k, 3 * h, head_in,
                         prob.data_ptr(), s, (self.heads * s * s, s * s), alpha=1.0 / math.sqrt(d))
        hip.softmax_fwd(prob, hip.MASK_CODES[mask], ctx.key_len if mask == "key_padding" else None, stream=ctx.stream)
        if drop is not None:
            # the stash keeps the probabilities themselves (the softmax backward needs them); V meets the dropped-out copy
            kept = ctx.buf("prob_drop", tuple(prob.shape))
            hip.dropout_apply(prob, kept, drop[0], drop[1], stream=ctx.stream)
            prob = kept
        # ctx = P V, written straight into the [rows, hidden] layout (head j -> columns j*d..)
        self._heads_gemm(ctx, hip.NN, s, d, s, prob.data_ptr(), s, (self.heads * s * s, s * s), v, 3 * h, head_in,
                         st["ctx"].data_ptr(), h, (s * h, d))

    def _attention_bwd(self, d_ctx, d_qkv, st, ctx, site=0, mask=None):
        h, d, s = self.hidden, self.head_dim, ctx.seq
        mask = self.mask if mask is None else mask
        drop = self._drop(ctx, site)
        if self.fused_attention(ctx):
            delta = ctx.buf("attn_delta", (ctx.batch, self.heads, s))
            hip.attention_bwd(st["qkv"], st["ctx"], d_ctx, st["lse"], delta, d_qkv, ctx.batch, self.heads, s,
                              hip.MASK_CODES[mask], ctx.key_len if mask == "key_padding" else None, stream=ctx.stream,
                              dropout=drop)
            return
        es = st["qkv"].element_size()
        q = st["qkv"].data_ptr()
        k, v = q + h * es, q + 2 * h * es
        dq = d_qkv.data_ptr()
        dk, dv = dq + h * es, dq + 2 * h * es
        head_in, head_ctx, head_p = (s * 3 * h, d), (s * h, d), (self.heads * s * s, s * s)
        prob = st["prob"]
        d_prob = ctx.buf("d_prob", tuple(prob.shape))
        scale = 1.0 / math.sqrt(d)
        # dV = P~^T dctx, P~ = what multiplied V in the forward (the dropped-out probabilities, made again)
        p_fwd = prob
        if drop is not None:
            p_fwd = ctx.buf("prob_drop", tuple(prob.shape))
            hip.dropout_apply(prob, p_fwd, drop[0], drop[1], stream=ctx.stream)
        self._heads_gemm(ctx, hip.TN, s, d, s, p_fwd.data_ptr(), s, head_p, d_ctx.data_ptr(), h, head_ctx,
                         dv, 3 * h, head_in)
        # dP~ = dctx V^T ; dP = dropout'(dP~) ; dS = P * (dP - rowsum(dP * P))
        self._heads_gemm(ctx, hip.NT, s, s, d, d_ctx.data_ptr(), h, head_ctx, v, 3 * h, head_in,
                         d_prob.data_ptr(), s, head_p)
        if drop is not None:
            hip.dropout_apply(d_prob, d_prob, drop[0], drop[1], stream=ctx.stream)
        hip.softmax_bwd(prob, d_prob, stream=ctx.stream)
        # dQ = dS K / sqrt(d) ; dK = dS^T Q / sqrt(d)
        self._heads_gemm(ctx, hip.NN, s, d, s, d_prob.data_ptr(), s, head_p, k, 3 * h, head_in,
                         dq, 3 * h, head_in, alpha=scale)
        self._heads_gemm(ctx, hip.TN, s, d, s, d_prob.data_ptr(), s, head_p, q, 3 * h, head_in,
                         dk, 3 * h, head_in, alpha=scale)

    # ------------------------------------------------------------------ forward / backward
    def forward(self, x, st, ctx):
        """x: [rows, hidden] (kept by reference in the stash); returns st['out']."""
        w, sm = self.w, ctx.stream
        kind, act = hip.LN_CODES[self.ln], hip.ACT_CODES[self.activation]
        st["x0"] = x
        hip.layernorm_fwd(x, w["sublayer.0.norm.a_2"], w["sublayer.0.norm.b_2"], st["n1"], st["mean1"],
                          st["rinv1"], kind, self.eps, stream=sm)
        ctx.gemm(hip.NT, st["n1"], w["qkv.weight"], st["qkv"], bias=w["qkv.bias"], stream=sm)
        self._attention_fwd(st, ctx)
        ctx.gemm(hip.NT, st["ctx"], w["self_attn.linears.3.weight"], st["x1"], bias=w["self_attn.linears.3.bias"],
                 epilogue=hip.EPI_RESIDUAL, resid=x, dropout=self._drop(ctx, self.SITE_SUBLAYER0), stream=sm)
        hip.layernorm_fwd(st["x1"], w["sublayer.1.norm.a_2"], w["sublayer.1.norm.b_2"], st["n2"], st["mean2"],
                          st["rinv2"], kind, self.eps, stream=sm)
        # activation and its derivative (kept for the backward pass, which then multiplies instead of
        # evaluating act') both leave the GEMM epilogue: on the power-limited stage the saved pass over the
        # pre-activation (read 64 MB, write 64 MB at the GPT-2-medium shapes) outweighs the epilogue's
        # transcendental work (measured inside the stage, not on the kernel alone)
        if ctx.defer or self.activation == "relu":
            # act' is read by the backward pass only: a forward that most likely has none writes act alone (and a
            # ReLU layer never writes it: its backward pass reads the derivative off act)
            ctx.gemm(hip.NT, st["n2"], w["feed_forward.w_1.weight"], st["act"], bias=w["feed_forward.w_1.bias"],
                     epilogue=hip.EPI_ACT, act=act, dropout=self._drop(ctx, self.SITE_FFN), stream=sm)
        else:
            self._ffn1(st, ctx)
        ctx.gemm(hip.NT, st["act"], w["feed_forward.w_2.weight"], st["out"], bias=w["feed_forward.w_2.bias"],
                 epilogue=hip.EPI_RESIDUAL, resid=st["x1"], dropout=self._drop(ctx, self.SITE_SUBLAYER1), stream=sm)
        return st["out"]

    def _ffn1(self, st, ctx):
        """act and act' of the feed-forward's hidden layer; under dropout both carry the keep factor, so the backward
        pass multiplies by the stored derivative as before."""
        w = self.w
        ctx.gemm(hip.NT, st["n2"], w["feed_forward.w_1.weight"], st["act"], bias=w["feed_forward.w_1.bias"],
                 epilogue=hip.EPI_ACT_DACT, act=hip.ACT_CODES[self.activation], aux_out=st["dact"],
                 dropout=self._drop(ctx, self.SITE_FFN), stream=ctx.stream)

    def backward(self, d_out, d_x, st, ctx):
        """d_out: gradient of st['out']; writes the input gradient into d_x; parameter
        gradients are accumulated (fp32)."""
        w, g, sm, ws = self.w, self.g, ctx.stream, ctx.workspace
        R, h, f = ctx.rows, self.hidden, self.ffn
        kind, act = hip.LN_CODES[self.ln], hip.ACT_CODES[self.activation]
        d_ffn, d_h0, d_h1 = ctx.buf("d_ffn", (R, f)), ctx.buf("d_h0", (R, h)), ctx.buf("d_h1", (R, h))
        d_qkv = ctx.buf("d_qkv", (R, 3 * h))
        # weight gradients dW += dy^T x are collected and issued as one grouped launch at the end:
        # each alone has too few output tiles to fill the GPU
        wgrads = []
        # ... and each carries its bias gradient (column sums of dy) in the same kernel
        wgrad = lambda dy, x, name: wgrads.append(hip.gemm_desc(
            hip.TN, dy, x, g[name], accumulate=True, colsum_out=g[name[:-len("weight")] + "bias"], colsum_ws=ws))
        if ctx.deferred and self.activation != "relu":
            self._ffn1(st, ctx)   # the forward of this stash left act' out: same kernel, same bits as a normal forward
        # the gradient behind a sublayer's dropout feeds the sublayer; the residual branch takes the one in front of it
        d_ff2, d_proj = d_out, None
        if self.dropout > 0:
            d_ff2 = ctx.buf("d_drop1", (R, h))
            hip.dropout_apply(d_out, d_ff2, *self._drop(ctx, self.SITE_SUBLAYER1), stream=sm)
        # feed-forward
        wgrad(d_ff2, st["act"], "feed_forward.w_2.weight")
        if self.activation == "relu":
            # act = relu(u) * keep / (1 - p): positive exactly where the gradient passes, and then with factor 1 / (1 - p)
            ctx.gemm(hip.NN, d_ff2, w["feed_forward.w_2.weight"], d_ffn, epilogue=hip.EPI_MUL_POS, aux_in=st["act"],
                     alpha=1.0 / (1.0 - self.dropout) if self.dropout > 0 else 1.0, stream=sm)
        else:
            ctx.gemm(hip.NN, d_ff2, w["feed_forward.w_2.weight"], d_ffn, epilogue=hip.EPI_MUL, aux_in=st["dact"], stream=sm)
        wgrad(d_ffn, st["n2"], "feed_forward.w_1.weight")
        ctx.gemm(hip.NN, d_ffn, w["feed_forward.w_1.weight"], d_h0, stream=sm)
        # d_x1 = d_out + LN2'(d_n2)
        hip.layernorm_bwd(st["x1"], w["sublayer.1.norm.a_2"], st["mean2"], st["rinv2"], d_h0, d_out, d_h1,
                          g["sublayer.1.norm.a_2"], g["sublayer.1.norm.b_2"], ws, kind, self.eps, stream=sm)
        # attention output projection
        d_proj = d_h1
        if self.dropout > 0:
            d_proj = ctx.buf("d_drop0", (R, h))
            hip.dropout_apply(d_h1, d_proj, *self._drop(ctx, self.SITE_SUBLAYER0), stream=sm)
        wgrad(d_proj, st["ctx"], "self_attn.linears.3.weight")
        ctx.gemm(hip.NN, d_proj, w["self_attn.linears.3.weight"], d_h0, stream=sm)
        self._attention_bwd(d_h0, d_qkv, st, ctx)
        # QKV projection
        wgrad(d_qkv, st["n1"], "qkv.weight")
        ctx.gemm(hip.NN, d_qkv, w["qkv.weight"], d_h0, stream=sm)
        # d_x0 = d_x1 + LN1'(d_n1)
        hip.layernorm_bwd(st["x0"], w["sublayer.0.norm.a_2"], st["mean1"], st["rinv1"], d_h0, d_h1, d_x,
                          g["sublayer.0.norm.a_2"], g["sublayer.0.norm.b_2"], ws, kind, self.eps, stream=sm)
        # d_out (d_drop1), d_ffn, d_h1 (d_drop0) and d_qkv still hold the four output gradients here
        ctx.gemm_grouped(wgrads, stream=sm)
        return d_x


class DecoderLayer(TransformerLayer):
    """The layer of the reference's GPT-2 script, ``DecoderLayerSimple`` (DeepSpeedExamples/pipeline_parallelism/
    gpt2.py:20-34): three pre-LN residual sublayers -- self-attention, attention over a "memory" (queries from the
    normalised stream, keys and values from ``m = sqrt(1 - x)`` of the layer's own INPUT ``x``: the script has no second
    input, gpt2.py:31), feed-forward.  ``m`` is defined for inputs below 1; beyond, its NaN enters the attention as
    in the reference (what becomes of NaN scores inside the attention kernels is not specified here).

    Parameters carry the reference module's names: ``self_attn.linears.{0..3}``, ``src_attn.linears.{0..3}``,
    ``feed_forward.w_{1,2}``, ``sublayer.{0,1,2}.norm.{a_2,b_2}``.  The memory attention reuses the kernels of
    the self-attention: its queries (one product on the normalised stream) and its keys / values (one product on
    ``m``, the two weights being neighbours in the arena) are written side by side into one ``[rows, 3h]`` buffer.
    Dropout sites: the four of :class:`TransformerLayer` (0 self-attention probabilities, 1 first sublayer, 2
    feed-forward hidden, 3 last sublayer) plus 4 (memory-attention probabilities) and 5 (second sublayer).
    ``mask`` applies to the self-attention only (the script passes none)."""

    SITE_SRC_ATTENTION, SITE_SUBLAYER_SRC = 4, 5

    REFERENCE_ORDER = tuple(
        [f"self_attn.linears.{i}.{k}" for i in range(4) for k in ("weight", "bias")] +
        [f"src_attn.linears.{i}.{k}" for i in range(4) for k in ("weight", "bias")] +
        ["feed_forward.w_1.weight", "feed_forward.w_1.bias", "feed_forward.w_2.weight", "feed_forward.w_2.bias"] +
        [f"sublayer.{i}.norm.{k}" for i in range(3) for k in ("a_2", "b_2")])

    def param_specs(self):
        h, f = self.hidden, self.ffn
        return OrderedDict([
            ("sublayer.0.norm.a_2", (h,)), ("sublayer.0.norm.b_2", (h,)),
            ("self_attn.linears.0.weight", (h, h)), ("self_attn.linears.1.weight", (h, h)), ("self_attn.linears.2.weight", (h, h)),
            ("self_attn.linears.0.bias", (h,)), ("self_attn.linears.1.bias", (h,)), ("self_attn.linears.2.bias", (h,)),
            ("self_attn.linears.3.weight", (h, h)), ("self_attn.linears.3.bias", (h,)),
            ("sublayer.1.norm.a_2", (h,)), ("sublayer.1.norm.b_2", (h,)),
            ("src_attn.linears.0.weight", (h, h)), ("src_attn.linears.0.bias", (h,)),
            ("src_attn.linears.1.weight", (h, h)), ("src_attn.linears.2.weight", (h, h)),      # keys, values: one [2h, h] product
            ("src_attn.linears.1.bias", (h,)), ("src_attn.linears.2.bias", (h,)),
            ("src_attn.linears.3.weight", (h, h)), ("src_attn.linears.3.bias", (h,)),
            ("sublayer.2.norm.a_2", (h,)), ("sublayer.2.norm.b_2", (h,)),
            ("feed_forward.w_1.weight", (f, h)), ("feed_forward.w_1.bias", (f,)),
            ("feed_forward.w_2.weight", (h, f)), ("feed_forward.w_2.bias", (h,)),
        ])

    def init_params(self, master, seed):
        """Weights N(0, init_std) from per-tensor seeded generators (index = position in the reference module's
        parameter order), biases 0, LayerNorm gain 1."""
        for i, name in enumerate(self.REFERENCE_ORDER):
            t = master[name]
            if name.endswith("a_2"):
                t.fill_(1.0)
            elif name.endswith("weight"):
                g = torch.Generator().manual_seed(seed * 1000 + i)
                t.copy_(torch.randn(t.shape, generator=g, dtype=torch.float32) * self.init_std)
            else:
                t.zero_()

    def bind(self, compute, grads):
        super().bind(compute, grads)
        h = self.hidden
        for d, src in ((self.w, compute), (self.g, grads)):
            d["kv.weight"] = torch.as_strided(src["src_attn.linears.1.weight"], (2 * h, h), (h, 1))
            d["kv.bias"] = torch.as_strided(src["src_attn.linears.1.bias"], (2 * h,), (1,))

    def stash_specs(self, ctx):
        R, h, f = ctx.rows, self.hidden, self.ffn
        dt, f32 = ctx.dtype, torch.float32
        fused = self.fused_attention(ctx)
        attn = lambda tag: (f"lse{tag}", (ctx.batch, self.heads, ctx.seq), f32) if fused else \
            (f"prob{tag}", (ctx.batch, self.heads, ctx.seq, ctx.seq), dt)
        dact = [] if self.activation == "relu" else [("dact", (R, f), dt)]
        return [
            ("n1", (R, h), dt), ("qkv", (R, 3 * h), dt), attn(""), ("ctx", (R, h), dt), ("x1", (R, h), dt),
            ("mem", (R, h), dt), ("n_src", (R, h), dt), ("qkv_src", (R, 3 * h), dt), attn("_src"), ("ctx_src", (R, h), dt),
            ("x2", (R, h), dt), ("n2", (R, h), dt), *dact, ("act", (R, f), dt), ("out", (R, h), dt),
            ("mean1", (R,), f32), ("rinv1", (R,), f32), ("mean_src", (R,), f32), ("rinv_src", (R,), f32),
            ("mean2", (R,), f32), ("rinv2", (R,), f32),
        ]

    def scratch_specs(self, ctx):
        R, h = ctx.rows, self.hidden
        specs = super().scratch_specs(ctx) + [("d_mem", (R, h), ctx.dtype), ("d_h2", (R, h), ctx.dtype)]
        if self.dropout > 0:
            specs.append(("d_drop_src", (R, h), ctx.dtype))
        return specs

    def flops_fwd(self, batch, seq):
        h, f = self.hidden, self.ffn
        return batch * seq * (16 * h * h + 4 * h * f) + 8 * batch * seq * seq * h

    def _src_views(self, st):
        return {"qkv": st["qkv_src"], "ctx": st["ctx_src"], "lse": st.get("lse_src"), "prob": st.get("prob_src")}

    def forward(self, x, st, ctx):
        w, sm = self.w, ctx.stream
        kind, act = hip.LN_CODES[self.ln], hip.ACT_CODES[self.activation]
        h = self.hidden
        st["x0"] = x
        hip.sqrt_one_minus_fwd(x, st["mem"], stream=sm)                                      # gpt2.py:31
        # sublayer 0: self-attention
        hip.layernorm_fwd(x, w["sublayer.0.norm.a_2"], w["sublayer.0.norm.b_2"], st["n1"], st["mean1"], st["rinv1"],
                          kind, self.eps, stream=sm)
        ctx.gemm(hip.NT, st["n1"], w["qkv.weight"], st["qkv"], bias=w["qkv.bias"], stream=sm)
        self._attention_fwd(st, ctx, site=self.SITE_ATTENTION)
        ctx.gemm(hip.NT, st["ctx"], w["self_attn.linears.3.weight"], st["x1"], bias=w["self_attn.linears.3.bias"],
                 epilogue=hip.EPI_RESIDUAL, resid=x, dropout=self._drop(ctx, self.SITE_SUBLAYER0), stream=sm)
        # sublayer 1: queries from the stream, keys and values from the memory
        hip.layernorm_fwd(st["x1"], w["sublayer.1.norm.a_2"], w["sublayer.1.norm.b_2"], st["n_src"], st["mean_src"],
                          st["rinv_src"], kind, self.eps, stream=sm)
        qs = st["qkv_src"]
        ctx.gemm(hip.NT, st["n_src"], w["src_attn.linears.0.weight"], qs[:, :h], bias=w["src_attn.linears.0.bias"], stream=sm)
        ctx.gemm(hip.NT, st["mem"], w["kv.weight"], qs[:, h:], bias=w["kv.bias"], stream=sm)
        self._attention_fwd(self._src_views(st), ctx, site=self.SITE_SRC_ATTENTION, mask="none")
        ctx.gemm(hip.NT, st["ctx_src"], w["src_attn.linears.3.weight"], st["x2"], bias=w["src_attn.linears.3.bias"],
                 epilogue=hip.EPI_RESIDUAL, resid=st["x1"], dropout=self._drop(ctx, self.SITE_SUBLAYER_SRC), stream=sm)
        # sublayer 2: feed-forward
        hip.layernorm_fwd(st["x2"], w["sublayer.2.norm.a_2"], w["sublayer.2.norm.b_2"], st["n2"], st["mean2"],
                          st["rinv2"], kind, self.eps, stream=sm)
        if ctx.defer or self.activation == "relu":
            ctx.gemm(hip.NT, st["n2"], w["feed_forward.w_1.weight"], st["act"], bias=w["feed_forward.w_1.bias"],
                     epilogue=hip.EPI_ACT, act=act, dropout=self._drop(ctx, self.SITE_FFN), stream=sm)
        else:
            self._ffn1(st, ctx)
        ctx.gemm(hip.NT, st["act"], w["feed_forward.w_2.weight"], st["out"], bias=w["feed_forward.w_2.bias"],
                 epilogue=hip.EPI_RESIDUAL, resid=st["x2"], dropout=self._drop(ctx, self.SITE_SUBLAYER1), stream=sm)
        return st["out"]

    def backward(self, d_out, d_x, st, ctx):
        w, g, sm, ws = self.w, self.g, ctx.stream, ctx.workspace
        R, h, f = ctx.rows, self.hidden, self.ffn
        kind = hip.LN_CODES[self.ln]
        d_ffn, d_h0, d_h1, d_h2 = (ctx.buf("d_ffn", (R, f)), ctx.buf("d_h0", (R, h)), ctx.buf("d_h1", (R, h)),
                                   ctx.buf("d_h2", (R, h)))
        d_qkv, d_mem = ctx.buf("d_qkv", (R, 3 * h)), ctx.buf("d_mem", (R, h))
        wgrads = []
        wgrad = lambda dy, x, name, bias=None: wgrads.append(hip.gemm_desc(
            hip.TN, dy, x, g[name], accumulate=True, colsum_out=g[bias or (name[:-len("weight")] + "bias")], colsum_ws=ws))

        def flush():
            # the weight gradients collected so far, before a scratch buffer they read is written again
            if wgrads:
                ctx.gemm_grouped(list(wgrads), stream=sm)
                wgrads.clear()
        if ctx.deferred and self.activation != "relu":
            self._ffn1(st, ctx)
        # ---- sublayer 2: feed-forward (as in TransformerLayer.backward)
        d_ff2 = d_out
        if self.dropout > 0:
            d_ff2 = ctx.buf("d_drop1", (R, h))
            hip.dropout_apply(d_out, d_ff2, *self._drop(ctx, self.SITE_SUBLAYER1), stream=sm)
        wgrad(d_ff2, st["act"], "feed_forward.w_2.weight")
        if self.activation == "relu":
            ctx.gemm(hip.NN, d_ff2, w["feed_forward.w_2.weight"], d_ffn, epilogue=hip.EPI_MUL_POS, aux_in=st["act"],
                     alpha=1.0 / (1.0 - self.dropout) if self.dropout > 0 else 1.0, stream=sm)
        else:
            ctx.gemm(hip.NN, d_ff2, w["feed_forward.w_2.weight"], d_ffn, epilogue=hip.EPI_MUL, aux_in=st["dact"], stream=sm)
        wgrad(d_ffn, st["n2"], "feed_forward.w_1.weight")
        ctx.gemm(hip.NN, d_ffn, w["feed_forward.w_1.weight"], d_h0, stream=sm)
        # d_x2 = d_out + LN2'(d_n2)  -> d_h2
        hip.layernorm_bwd(st["x2"], w["sublayer.2.norm.a_2"], st["mean2"], st["rinv2"], d_h0, d_out, d_h2,
                          g["sublayer.2.norm.a_2"], g["sublayer.2.norm.b_2"], ws, kind, self.eps, stream=sm)
        # ---- sublayer 1: attention over the memory
        d_proj = d_h2
        if self.dropout > 0:
            d_proj = ctx.buf("d_drop_src", (R, h))
            hip.dropout_apply(d_h2, d_proj, *self._drop(ctx, self.SITE_SUBLAYER_SRC), stream=sm)
        wgrad(d_proj, st["ctx_src"], "src_attn.linears.3.weight")
        ctx.gemm(hip.NN, d_proj, w["src_attn.linears.3.weight"], d_h0, stream=sm)
        self._attention_bwd(d_h0, d_qkv, self._src_views(st), ctx, site=self.SITE_SRC_ATTENTION, mask="none")
        wgrad(d_qkv[:, :h], st["n_src"], "src_attn.linears.0.weight")
        wgrads.append(hip.gemm_desc(hip.TN, d_qkv[:, h:], st["mem"], g["kv.weight"], accumulate=True,
                                    colsum_out=g["kv.bias"], colsum_ws=ws))
        ctx.gemm(hip.NN, d_qkv[:, :h], w["src_attn.linears.0.weight"], d_h0, stream=sm)        # d_n_src
        ctx.gemm(hip.NN, d_qkv[:, h:], w["kv.weight"], d_mem, stream=sm)                       # gradient of the memory
        # d_x1 = d_x2 + LN_src'(d_n_src)  -> d_h1
        hip.layernorm_bwd(st["x1"], w["sublayer.1.norm.a_2"], st["mean_src"], st["rinv_src"], d_h0, d_h2, d_h1,
                          g["sublayer.1.norm.a_2"], g["sublayer.1.norm.b_2"], ws, kind, self.eps, stream=sm)
        flush()      # d_qkv, d_ffn and the first sublayers' gradient buffers are free again
        # ---- sublayer 0: self-attention
        d_proj0 = d_h1
        if self.dropout > 0:
            d_proj0 = ctx.buf("d_drop0", (R, h))
            hip.dropout_apply(d_h1, d_proj0, *self._drop(ctx, self.SITE_SUBLAYER0), stream=sm)
        wgrad(d_proj0, st["ctx"], "self_attn.linears.3.weight")
        ctx.gemm(hip.NN, d_proj0, w["self_attn.linears.3.weight"], d_h0, stream=sm)
        self._attention_bwd(d_h0, d_qkv, st, ctx, site=self.SITE_ATTENTION)
        wgrad(d_qkv, st["n1"], "qkv.weight")
        ctx.gemm(hip.NN, d_qkv, w["qkv.weight"], d_h0, stream=sm)
        # d_x = d_x1 + LN0'(d_n1) + d_mem * dm/dx
        hip.layernorm_bwd(st["x0"], w["sublayer.0.norm.a_2"], st["mean1"], st["rinv1"], d_h0, d_h1, d_x,
                          g["sublayer.0.norm.a_2"], g["sublayer.0.norm.b_2"], ws, kind, self.eps, stream=sm)
        hip.sqrt_one_minus_bwd(d_mem, st["mem"], d_x, accumulate=True, stream=sm)
        flush()
        return d_x


class FinalLayerNorm:
    """A LayerNorm as a layer of its own: ``encoder.norm``, the first of the two layers that end the reference's
    transformer script (transformer.py:181,250).  Parameters ``a_2`` / ``b_2`` as in the reference's ``LayerNorm``
    module (transformer.py:77-88)."""

    REFERENCE_ORDER = ("a_2", "b_2")

    def __init__(self, hidden, ln="annotated", ln_eps=None):
        if ln not in hip.LN_CODES:
            raise ValueError(f"unsupported LayerNorm kind {ln}")
        self.hidden, self.ln = hidden, ln
        self.eps = ln_eps if ln_eps is not None else (1e-6 if ln == "annotated" else 1e-5)
        self.w = self.g = None

    feature_dim = property(lambda self: self.hidden)
    out_features = property(lambda self: self.hidden)

    def param_specs(self):
        return OrderedDict([("a_2", (self.hidden,)), ("b_2", (self.hidden,))])

    def num_params(self):
        return 2 * self.hidden

    def init_params(self, master, seed):
        master["a_2"].fill_(1.0)
        master["b_2"].zero_()

    def bind(self, compute, grads):
        self.w, self.g = dict(compute), dict(grads)

    def stash_specs(self, ctx):
        R, f32 = ctx.rows, torch.float32
        return [("out", (R, self.hidden), ctx.dtype), ("mean", (R,), f32), ("rinv", (R,), f32)]

    def scratch_specs(self, ctx):
        return []

    def workspace_elems(self):
        return hip.layernorm_bwd_workspace(self.hidden)

    def flops_fwd(self, batch, seq):
        return 0

    def forward(self, x, st, ctx):
        st["x0"] = x
        hip.layernorm_fwd(x, self.w["a_2"], self.w["b_2"], st["out"], st["mean"], st["rinv"], hip.LN_CODES[self.ln],
                          self.eps, stream=ctx.stream)
        return st["out"]

    def backward(self, d_out, d_x, st, ctx):
        hip.layernorm_bwd(st["x0"], self.w["a_2"], st["mean"], st["rinv"], d_out, None, d_x, self.g["a_2"], self.g["b_2"],
                          ctx.workspace, hip.LN_CODES[self.ln], self.eps, stream=ctx.stream)
        return d_x


class SumLast:
    """``lambda x: x.sum(-1)``: the parameter-free layer that ends the reference's transformer script
    (transformer.py:250); ``[rows, hidden] -> [rows, 1]``, so that ``MSELoss`` compares with ``[batch, seq]`` labels
    (transformer.py:205-219,264)."""

    REFERENCE_ORDER = ()

    def __init__(self, hidden):
        self.hidden = hidden

    feature_dim = property(lambda self: self.hidden)
    out_features = 1

    def param_specs(self):
        return OrderedDict()

    def num_params(self):
        return 0

    def init_params(self, master, seed):
        pass

    def bind(self, compute, grads):
        pass

    def stash_specs(self, ctx):
        return [("out", (ctx.rows, 1), ctx.dtype)]

    def scratch_specs(self, ctx):
        return []

    def workspace_elems(self):
        return 0

    def flops_fwd(self, batch, seq):
        return 0

    def forward(self, x, st, ctx):
        hip.rowsum_fwd(x, st["out"], stream=ctx.stream)
        return st["out"]

    def backward(self, d_out, d_x, st, ctx):
        hip.rowsum_bwd(d_out, d_x, stream=ctx.stream)
        return d_x


class BottleNeck:
    """ResNet bottleneck block ``ReLU(BN(conv1x1(ReLU(BN(conv3x3(ReLU(BN(conv1x1 x)))))) + shortcut(x))`` (reference
    ``BottleNeck``, DeepSpeedExamples/pipeline_parallelism/resnet.py:49-75) on NHWC activations viewed as
    ``[rows = N*H*W, channels]``.  The shortcut is the identity when ``stride == 1`` and ``in_channels == 4 *
    out_channels``, else ``BN(conv1x1(x, stride))`` (resnet.py:68-72); ``stride`` sits on the 3x3 convolution
    (resnet.py:58), so a down-sampling block turns ``N*H*W`` input rows into ``N*ceil(H/s)*ceil(W/s)`` output rows.
    The 1x1 convolutions are plain GEMMs on the row view (the strided one on the rows of every s-th pixel,
    ``hip.subsample``); the 3x3 convolution with stride 1, its input gradient (``hip.conv3x3``) and its weight
    gradient (``gemm_desc(..., conv=)``) are implicit GEMMs: the operand loader gathers the 3x3 neighbourhoods, no
    patch matrix is written.  Where the implicit kernels do not take the problem (a stride, fp32, channel counts that
    are not multiples of 64, resp. 128 for the weight gradient) the same products run as GEMMs over the gathered patch
    matrix ``[rows, 9*C]``.  Parameter names are the reference's; the 3x3 weight is kept as ``[out, 3, 3, in]``
    (tap-major, channel-minor) so that it is the ``[out, 9*in]`` GEMM operand as it lies in memory (the reference
    holds ``[out, in, 3, 3]``)."""

    EXPANSION = 4

    def __init__(self, in_channels, out_channels, stride=1, height=14, width=14, bn_eps=1e-5, bn_momentum=0.1):
        if stride not in (1, 2):
            raise NotImplementedError(f"bottleneck stride {stride}: the reference's ResNets use 1 and 2")
        self.cin, self.cmid, self.cout = in_channels, out_channels, self.EXPANSION * out_channels
        self.stride, self.h, self.w = stride, height, width
        self.projection = stride != 1 or in_channels != self.cout
        self.eps, self.momentum = bn_eps, bn_momentum
        self.w_ = self.g_ = None
        self.running = None
        self._stats_ok = {}    # (shapes, dtype) -> whether the GEMM of a 1x1 convolution leaves strip statistics

    @property
    def feature_dim(self):
        return self.cin

    @property
    def out_features(self):
        return self.cout

    def out_seq(self, seq):
        """Pixels per image behind the block, for ``seq`` in front of it."""
        if self.stride == 1:
            return seq
        h, w = self._image(seq)
        return ((h - 1) // self.stride + 1) * ((w - 1) // self.stride + 1)

    def param_specs(self):
        ci, cm, co = self.cin, self.cmid, self.cout
        specs = [("residual_function.0.weight", (cm, ci)),
                 ("residual_function.1.weight", (cm,)), ("residual_function.1.bias", (cm,)),
                 ("residual_function.3.weight", (cm, 3, 3, cm)),
                 ("residual_function.4.weight", (cm,)), ("residual_function.4.bias", (cm,)),
                 ("residual_function.6.weight", (co, cm)),
                 ("residual_function.7.weight", (co,)), ("residual_function.7.bias", (co,))]
        if self.projection:
            specs += [("shortcut.0.weight", (co, ci)), ("shortcut.1.weight", (co,)), ("shortcut.1.bias", (co,))]
        return OrderedDict(specs)

    def num_params(self):
        return sum(math.prod(s) for s in self.param_specs().values())

    # registration order of the reference's ``residual_function`` and ``shortcut`` (resnet.py:55-72)
    RESIDUAL_ORDER = ("residual_function.0.weight", "residual_function.1.weight", "residual_function.1.bias",
                      "residual_function.3.weight", "residual_function.4.weight", "residual_function.4.bias",
                      "residual_function.6.weight", "residual_function.7.weight", "residual_function.7.bias")
    SHORTCUT_ORDER = ("shortcut.0.weight", "shortcut.1.weight", "shortcut.1.bias")
    _CONV1X1 = ("residual_function.0.weight", "residual_function.6.weight", "shortcut.0.weight")

    @property
    def REFERENCE_ORDER(self):
        return self.RESIDUAL_ORDER + (self.SHORTCUT_ORDER if self.projection else ())

    @staticmethod
    def to_native(name, tensor):
        """Reference layout -> arena layout: conv weights [O, I, kh, kw] -> [O, kh, kw, I]."""
        if tensor.dim() == 4:
            t = tensor.permute(0, 2, 3, 1).contiguous()
            return t.view(t.shape[0], -1) if t.shape[1] == 1 else t
        return tensor

    @classmethod
    def to_reference(cls, name, tensor):
        """Arena layout -> the reference's: 1x1 convolutions [O, I] -> [O, I, 1, 1], the 3x3 one [O, kh, kw, I] ->
        [O, I, kh, kw] (a copy)."""
        if name in cls._CONV1X1:
            return tensor.reshape(tensor.shape[0], tensor.shape[1], 1, 1)
        if name == "residual_function.3.weight":
            return tensor.permute(0, 3, 1, 2).contiguous()
        return tensor

    def init_params(self, master, seed):
        """He-normal convolution weights (std = sqrt(2 / fan_in)) from per-tensor seeded generators drawn in
        the reference's [O, I, kh, kw] layout, BN gain 1 / shift 0."""
        ref_shapes = {"residual_function.0.weight": (self.cmid, self.cin, 1, 1),
                      "residual_function.3.weight": (self.cmid, self.cmid, 3, 3),
                      "residual_function.6.weight": (self.cout, self.cmid, 1, 1),
                      "shortcut.0.weight": (self.cout, self.cin, 1, 1)}
        for i, name in enumerate(self.param_specs()):
            t = master[name]
            if name in ref_shapes:
                shape = ref_shapes[name]
                g = torch.Generator().manual_seed(seed * 1000 + i)
                wt = torch.randn(shape, generator=g, dtype=torch.float32) * math.sqrt(2.0 / (shape[1] * shape[2] * shape[3]))
                t.copy_(self.to_native(name, wt).view(t.shape))
            elif name.endswith("weight"):
                t.fill_(1.0)
            else:
                t.zero_()

    def bind(self, compute, grads):
        self.w_, self.g_ = dict(compute), dict(grads)
        for d in (self.w_, self.g_):
            d["conv2"] = d["residual_function.3.weight"].view(self.cmid, 9 * self.cmid)

    # ---------------------------------------------------------------- shapes
    def _image(self, seq):
        """(height, width) of the input image; a block taken over from a module does not know them: square
        images, side = sqrt(positions)."""
        if self.h is None or self.w is None:
            side = math.isqrt(seq)
            if side * side != seq:
                raise hip.HipKernelError(f"cannot infer a square image from {seq} positions: pass height= and width=")
            return side, side
        return self.h, self.w

    def _bind_image(self, ctx):
        self.h, self.w = self._image(ctx.seq)
        if ctx.seq != self.h * self.w:
            raise hip.HipKernelError(f"activation has {ctx.seq} positions, the block expects {self.h}x{self.w}")

    def _rows(self, ctx):
        """(input rows, output rows, output height, output width)."""
        self._bind_image(ctx)
        ho, wo = (self.h - 1) // self.stride + 1, (self.w - 1) // self.stride + 1
        return ctx.batch * self.h * self.w, ctx.batch * ho * wo, ho, wo

    def stash_specs(self, ctx):
        R, R2, _, _ = self._rows(ctx)
        cm, co = self.cmid, self.cout
        dt, f32 = ctx.dtype, torch.float32
        specs = [("y1", (R, cm), dt), ("a1", (R, cm), dt), ("y2", (R2, cm), dt), ("a2", (R2, cm), dt),
                 ("y3", (R2, co), dt), ("out", (R2, co), dt),
                 ("mean1", (cm,), f32), ("rstd1", (cm,), f32), ("mean2", (cm,), f32), ("rstd2", (cm,), f32),
                 ("mean3", (co,), f32), ("rstd3", (co,), f32)]
        if self.projection:
            specs += [("ys", (R2, co), dt), ("mean_s", (co,), f32), ("rstd_s", (co,), f32)]
        return specs

    def _wgrad_elems(self):
        n = self.cin * self.cmid + 9 * self.cmid * self.cmid + self.cmid * self.cout
        return n + (self.cout * self.cin if self.projection else 0)

    def scratch_specs(self, ctx):
        R, R2, _, _ = self._rows(ctx)
        ci, cm, co = self.cin, self.cmid, self.cout
        dt = ctx.dtype
        specs = [("d_col", (R2, 9 * cm), dt), ("d_y3", (R2, co), dt), ("d_res", (R2, co), dt),
                 ("d_m0", (R, cm), dt), ("d_m1", (R2, cm), dt), ("d_m2", (R, cm), dt),
                 # split-K partial products of the weight gradients (8 chunks of each, fp32)
                 ("splitk", (8 * self._wgrad_elems(),), torch.float32),
                 # backward sums of an inner BatchNorm per 32-row strip, left by the kernel that produces its gradient
                 ("bn_strips", (hip.bn_bwd_strips_workspace(R, cm),), torch.float32),
                 # the same for the last BatchNorm, left by the block behind this one (grad_sink)
                 ("bn_strips_in", (hip.bn_bwd_strips_workspace(R2, co),), torch.float32)]
        if self.projection:
            specs += [("d_ys", (R2, co), dt), ("d_xs", (R2, ci), dt)]
        return specs + self.forward_scratch_specs(ctx)

    def forward_scratch_specs(self, ctx):
        R, R2, _, _ = self._rows(ctx)
        specs = [("col", (R2, 9 * self.cmid), ctx.dtype),
                 ("strips", (hip.strip_stats_workspace(R, self.cout),), torch.float32)]
        if self.projection:
            specs += [("sc", (R2, self.cout), ctx.dtype), ("xs", (R2, self.cin), ctx.dtype)]
        return specs

    def workspace_elems(self):
        c = max(self.cin, self.cout)
        return max(hip.bn_workspace(c), hip.colsum_workspace(c))

    def flops_fwd(self, batch, seq):
        out = batch * self.out_seq(seq)
        f = 2 * batch * seq * self.cin * self.cmid + 2 * out * (9 * self.cmid * self.cmid + self.cmid * self.cout)
        return f + (2 * out * self.cin * self.cout if self.projection else 0)

    # ---------------------------------------------------------------- pieces
    _BN_NAMES = {1: "residual_function.1", 4: "residual_function.4", 7: "residual_function.7", "shortcut": "shortcut.1"}

    def _running(self, device):
        if self.running is None:
            z = lambda n, v: torch.full((n,), v, dtype=torch.float32, device=device)
            widths = [(1, self.cmid), (4, self.cmid), (7, self.cout)] + ([("shortcut", self.cout)] if self.projection else [])
            self.running = {i: (z(n, 0.0), z(n, 1.0)) for i, n in widths}
            for i, (m, v) in getattr(self, "adopted_running", {}).items():   # statistics of the module the block came from
                self.running[i][0].copy_(m)
                self.running[i][1].copy_(v)
        return self.running

    def _bn_fwd(self, idx, x, resid, y, mean, rstd, relu, ctx, strips=None):
        run = (None, None) if ctx.redundant else self._running(x.device)[idx]
        name = self._BN_NAMES[idx]
        hip.batchnorm_fwd(x, self.w_[f"{name}.weight"], self.w_[f"{name}.bias"],
                          resid, y, mean, rstd, run[0], run[1], ctx.workspace, self.eps, self.momentum, relu,
                          stream=ctx.stream, strip_stats=strips)

    def _conv1x1(self, x, weight, y, ctx):
        """1x1 convolution = GEMM on the NHWC rows; where the kernel can, it also leaves the strip statistics of
        its output for the BatchNorm that follows (returned, else None: that BatchNorm then reads y for them)."""
        strips = None
        key = (tuple(x.shape), tuple(weight.shape), x.dtype)
        if key not in self._stats_ok:
            self._stats_ok[key] = x.shape[0] <= 8192 and hip.gemm_strip_stats_supported(hip.NT, x, weight, y)
        if self._stats_ok[key]:
            strips = ctx.buf("strips", (hip.strip_stats_workspace(x.shape[0], y.shape[1]),))
        ctx.gemm(hip.NT, x, weight, y, stream=ctx.stream, strip_stats=strips)
        return strips

    def _implicit(self, ctx, mode):
        return self.stride == 1 and hip.conv3x3_supported(ctx.dtype, mode, ctx.batch, self.h, self.w, self.cmid, self.cmid)

    def _shortcut_input(self, x, ctx, R2):
        """Rows the projection shortcut reads: x itself, or the rows of every stride-th pixel."""
        if self.stride == 1:
            return x
        xs = ctx.buf("xs", (R2, self.cin))
        hip.subsample(x, xs, ctx.batch, self.h, self.w, self.cin, self.stride, stream=ctx.stream)
        return xs

    def forward(self, x, st, ctx):
        R, R2, _, _ = self._rows(ctx)
        w, sm, cm = self.w_, ctx.stream, self.cmid
        st["x0"] = x
        strips = self._conv1x1(x, w["residual_function.0.weight"], st["y1"], ctx)
        self._bn_fwd(1, st["y1"], None, st["a1"], st["mean1"], st["rstd1"], True, ctx, strips)
        if self._implicit(ctx, hip.CONV_FWD):
            strips = ctx.buf("strips", (hip.strip_stats_workspace(R, cm),)) if R <= 8192 else None
            ctx.conv3x3(hip.CONV_FWD, st["a1"], w["residual_function.3.weight"], st["y2"], ctx.batch, self.h, self.w,
                        cm, cm, strip_stats=strips, stream=sm)
        else:
            col = ctx.buf("col", (R2, 9 * cm))
            hip.patch3x3(st["a1"], col, ctx.batch, self.h, self.w, cm, stride=self.stride, stream=sm)
            strips = self._conv1x1(col, w["conv2"], st["y2"], ctx)
        self._bn_fwd(4, st["y2"], None, st["a2"], st["mean2"], st["rstd2"], True, ctx, strips)
        if self.projection:
            # the shortcut first: its normalised output is the residual the last BatchNorm adds before the ReLU
            sc = ctx.buf("sc", (R2, self.cout))
            strips = self._conv1x1(self._shortcut_input(x, ctx, R2), w["shortcut.0.weight"], st["ys"], ctx)
            self._bn_fwd("shortcut", st["ys"], None, sc, st["mean_s"], st["rstd_s"], False, ctx, strips)
        else:
            sc = x
        strips = self._conv1x1(st["a2"], w["residual_function.6.weight"], st["y3"], ctx)
        self._bn_fwd(7, st["y3"], sc, st["out"], st["mean3"], st["rstd3"], True, ctx, strips)
        return st["out"]

    def grad_sink(self, st, ctx):
        """What the layer behind this one may do to the gradient it hands over (``ctx.seq`` is this block's): mask it
        with the block's last ReLU and leave the backward sums of the last BatchNorm per strip -- the kernel that
        writes that gradient does both in its epilogue, this block's backward then starts without a reduction pass
        over its widest tensor.  None where the kernels for it do not exist (fp32)."""
        if ctx.dtype != torch.bfloat16:
            return None
        _, R2, _, _ = self._rows(ctx)
        return {"rows": R2, "cols": self.cout, "relu_out": st["out"], "x": st["y3"], "mean": st["mean3"], "rstd": st["rstd3"],
                "strips": ctx.buf("bn_strips_in", (hip.bn_bwd_strips_workspace(R2, self.cout),))}

    def backward(self, d_out, d_x, st, ctx):
        w, g, sm, ws = self.w_, self.g_, ctx.stream, ctx.workspace
        R, R2, _, _ = self._rows(ctx)
        ci, cm, co = self.cin, self.cmid, self.cout
        col = ctx.buf("col", (R2, 9 * cm))
        d_y3, d_res = ctx.buf("d_y3", (R2, co)), ctx.buf("d_res", (R2, co))
        d_m0, d_m1 = ctx.buf("d_m0", (R2, cm)), ctx.buf("d_m1", (R2, cm))

        def bn_strips(idx, xk, mk, rk, gk, strips, dx):
            name = self._BN_NAMES[idx]
            hip.batchnorm_bwd_strips(st[xk], w[f"{name}.weight"], st[mk], st[rk], gk, strips, dx,
                                     g[f"{name}.weight"], g[f"{name}.bias"], stream=sm)

        def bn(idx, xk, mk, rk, dy, relu_out, dx, g_out, strips_name):
            """BatchNorm backward with a reduction pass of its own.  bf16: the pass adds the sums up in the order of the
            GEMM epilogues that leave them elsewhere, so a gradient gives the same bits whichever kernel made its
            sums (a block at a stage or checkpoint-group boundary, a promoted stage, a shape the fused kernels do
            not take); the masked gradient goes to ``g_out``, else in place into ``dy``."""
            name = self._BN_NAMES[idx]
            if ctx.dtype != torch.bfloat16:
                hip.batchnorm_bwd(st[xk], w[f"{name}.weight"], st[mk], st[rk], dy, relu_out, dx, g_out,
                                  g[f"{name}.weight"], g[f"{name}.bias"], ws, stream=sm)
                return
            strips = ctx.buf(strips_name, (hip.bn_bwd_strips_workspace(*st[xk].shape),))
            masked = dy if relu_out is None else (g_out if g_out is not None else dy)
            hip.batchnorm_bwd_strip_sums(st[xk], st[mk], st[rk], dy, relu_out, masked if relu_out is not None else None, strips,
                                         stream=sm)
            bn_strips(idx, xk, mk, rk, masked, strips, dx)
        # final ReLU + BN3; d_res keeps the masked gradient for the shortcut
        if ctx.grad_presummed:
            # the block behind this one has masked d_out and left the sums (grad_sink)
            d_res = d_out
            bn_strips(7, "y3", "mean3", "rstd3", d_out, ctx.buf("bn_strips_in", (hip.bn_bwd_strips_workspace(R2, co),)), d_y3)
        else:
            bn(7, "y3", "mean3", "rstd3", d_out, st["out"], d_y3, d_res, "bn_strips_in")
        d_ys = d_xs = xs = None
        if self.projection:
            d_ys, d_xs = ctx.buf("d_ys", (R2, co)), ctx.buf("d_xs", (R2, ci))
            bn("shortcut", "ys", "mean_s", "rstd_s", d_res, None, d_ys, None, "bn_strips_in")
            ctx.gemm(hip.NN, d_ys, w["shortcut.0.weight"], d_xs, stream=sm)
            xs = self._shortcut_input(st["x0"], ctx, R2)
        # The two inner BatchNorms receive their gradient from a convolution's input gradient: where the kernel can,
        # it masks the gradient with the ReLU and leaves the normalisation's backward sums per strip, so that no
        # pass over the tensor is needed for them.
        key = ("bn_bwd", R2, cm, co, ctx.dtype)
        if key not in self._stats_ok:
            self._stats_ok[key] = hip.gemm_bn_bwd_supported(d_y3, w["residual_function.6.weight"], d_m0, st["a2"])
        if self._stats_ok[key]:
            strips = ctx.buf("bn_strips", (hip.bn_bwd_strips_workspace(R2, cm),))
            ctx.gemm_bn_bwd(d_y3, w["residual_function.6.weight"], d_m0, st["a2"], st["y2"], st["mean2"], st["rstd2"],
                            strips, stream=sm)                                             # d_a2, masked
            bn_strips(4, "y2", "mean2", "rstd2", d_m0, strips, d_m1)                       # d_y2
        else:
            ctx.gemm(hip.NN, d_y3, w["residual_function.6.weight"], d_m0, stream=sm)      # d_a2
            bn(4, "y2", "mean2", "rstd2", d_m0, st["a2"], d_m1, None, "bn_strips")         # d_y2
        # weight gradient of the 3x3 convolution: patch matrix gathered inside the GEMM, else built again here
        # (cheaper than stashing it)
        wgrad_implicit = (self._implicit(ctx, hip.CONV_DGRAD) and cm % 128 == 0 and R % 32 == 0 and 32 // self.w + 1 <= self.h)
        if not wgrad_implicit:
            hip.patch3x3(st["a1"], col, ctx.batch, self.h, self.w, cm, stride=self.stride, stream=sm)
        d_a1, d_m2 = ctx.buf("d_m0", (R, cm)), ctx.buf("d_m2", (R, cm))
        if self._implicit(ctx, hip.CONV_DGRAD):
            strips = ctx.buf("bn_strips", (hip.bn_bwd_strips_workspace(R, cm),))
            ctx.conv3x3_dgrad_bn(d_m1, w["residual_function.3.weight"], d_a1, ctx.batch, self.h, self.w, cm, cm,
                                 st["a1"], st["y1"], st["mean1"], st["rstd1"], strips, stream=sm)
            bn_strips(1, "y1", "mean1", "rstd1", d_a1, strips, d_m2)                       # d_y1
        else:
            d_col = ctx.buf("d_col", (R2, 9 * cm))
            ctx.gemm(hip.NN, d_m1, w["conv2"], d_col, stream=sm)
            hip.patch3x3(d_col, d_a1, ctx.batch, self.h, self.w, cm, adjoint=True, stride=self.stride, stream=sm)
            bn(1, "y1", "mean1", "rstd1", d_a1, st["a1"], d_m2, None, "bn_strips")         # d_y1
        if self.projection and self.stride > 1:
            ctx.gemm(hip.NN, d_m2, w["residual_function.0.weight"], d_x, stream=sm)
            hip.subsample(d_xs, d_x, ctx.batch, self.h, self.w, ci, self.stride, adjoint=True, stream=sm)
        else:
            resid = d_xs if self.projection else d_res
            sink = ctx.grad_sink
            if sink is not None and (sink["rows"], sink["cols"]) == (R, ci):
                key = ("sink", R, ci, cm, ctx.dtype)
                if key not in self._stats_ok:
                    self._stats_ok[key] = hip.gemm_bn_bwd_supported(d_m2, w["residual_function.0.weight"], d_x, sink["relu_out"], resid)
                if not self._stats_ok[key]:
                    sink = None
            else:
                sink = None
            if sink is not None:
                ctx.gemm_bn_bwd(d_m2, w["residual_function.0.weight"], d_x, sink["relu_out"], sink["x"], sink["mean"],
                                sink["rstd"], sink["strips"], resid=resid, stream=sm)
                ctx.grad_sink_used = True
            else:
                ctx.gemm(hip.NN, d_m2, w["residual_function.0.weight"], d_x, epilogue=hip.EPI_RESIDUAL, resid=resid, stream=sm)
        # the weight gradients in one launch: few output tiles over thousands of rows, cut along the rows
        descs = [hip.gemm_desc(hip.TN, d_y3, st["a2"], g["residual_function.6.weight"], accumulate=True),
                 hip.gemm_desc(hip.TN, d_m1, st["a1"], g["conv2"], accumulate=True, conv=(self.h, self.w))
                 if wgrad_implicit else hip.gemm_desc(hip.TN, d_m1, col, g["conv2"], accumulate=True),
                 hip.gemm_desc(hip.TN, d_m2, st["x0"], g["residual_function.0.weight"], accumulate=True)]
        if self.projection:
            descs.append(hip.gemm_desc(hip.TN, d_ys, xs, g["shortcut.0.weight"], accumulate=True))
        ctx.gemm_grouped(descs, stream=sm, splitk_ws=ctx.buf("splitk", (8 * self._wgrad_elems(),)))
        return d_x


class MSELoss:
    """``nn.MSELoss()`` of the reference scripts (transformer.py:264) as a fused HIP kernel that
    also yields the output gradient.  Used as ``loss_fn`` of a last stage, and by the in-process
    peer that stands in for the downstream stages."""

    def __call__(self, y, target, d_y, grad_scale, loss_out, accumulate, workspace, stream=None):
        hip.mse_fwd_bwd(y, target, d_y, grad_scale, loss_out, accumulate, workspace, stream=stream)
