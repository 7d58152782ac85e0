"""Checks at the full shapes of the benchmark configurations -- the GPT-2-medium stage (rows 8192, hidden 1024,
ffn 4096, 16 heads, seq 1024) and the GPT-2-1.5B stage (rows 4096, hidden 1600, ffn 6400, 25 heads, seq 1024:
1600 = 25 x 64 is no multiple of the 128- and 256-wide tiles) -- through properties that do not need a full CPU
run: bit-reproducibility, oracle values on sampled rows / heads, softmax normalisation, causality, RC
bit-exactness; plus one failover at the 1.5B layer shape against the CPU oracle, and the BERT-large stage's attention
(seq 512, ragged key lengths) against fp64 autograd on sampled heads.  (The ResNet stage's block shape is a case of
tests/test_gpu_stage.py::test_resnet_stage_matches_oracle_with_rc.)"""
import math

import numpy as np
import pytest
import torch

import bamboo_amd
from bamboo_amd import LayerSpec, PipelineModule, SeededActivationQueue, TransformerLayer
from oracle import adam as oadam
from oracle import layers as ol

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
MB, SEQ, HID, HEADS, FFN = 8, 1024, 1024, 16, 4096
ROWS = MB * SEQ
# GPT-2-1.5B stage
MB5, HID5, HEADS5, FFN5 = 4, 1600, 25, 6400
ROWS5 = MB5 * SEQ


def randn(*shape, seed=0, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=DEV) * scale).to(dtype)


def l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("layout,M,N,K", [
    (0, ROWS, FFN, HID), (0, ROWS, 3 * HID, HID), (0, ROWS, HID, FFN),
    (1, ROWS, HID, FFN), (1, ROWS, FFN, HID), (2, FFN, HID, ROWS), (2, HID, HID, ROWS),
    # every product of a GPT-2-1.5B layer: forward (NT), input gradients (NN), weight gradients (TN)
    (0, ROWS5, 3 * HID5, HID5), (0, ROWS5, HID5, HID5), (0, ROWS5, FFN5, HID5), (0, ROWS5, HID5, FFN5),
    (1, ROWS5, HID5, 3 * HID5), (1, ROWS5, HID5, HID5), (1, ROWS5, HID5, FFN5), (1, ROWS5, FFN5, HID5),
    (2, 3 * HID5, HID5, ROWS5), (2, HID5, HID5, ROWS5), (2, FFN5, HID5, ROWS5), (2, HID5, FFN5, ROWS5)])
def test_gemm_full_shapes_sampled(hiplib, layout, M, N, K):
    a_shape = (K, M) if layout == hiplib.TN else (M, K)
    b_shape = (N, K) if layout == hiplib.NT else (K, N)
    A, B = randn(*a_shape, seed=1), randn(*b_shape, seed=2, scale=0.05)
    C = torch.empty(M, N, dtype=torch.float32 if layout == hiplib.TN else torch.bfloat16, device=DEV)
    if layout == hiplib.TN:
        C.zero_()
    hiplib.gemm(layout, A, B, C, accumulate=layout == hiplib.TN)
    # sampled rows, always with the first and the last one (the edges of the first and the last tile)
    idx = torch.cat([torch.tensor([0, M - 1]), torch.randint(0, M, (46,), generator=torch.Generator().manual_seed(3))]).to(DEV)
    Ar = (A[:, idx].t() if layout == hiplib.TN else A[idx]).double()
    ref = Ar @ (B.double().t() if layout == hiplib.NT else B.double())
    assert l2(C[idx], ref) < 1e-2
    assert l2(C[idx][:, -64:], ref[:, -64:]) < 1e-2       # the last columns: a partly filled tile when N % 256 != 0
    C2 = torch.zeros_like(C)
    hiplib.gemm(layout, A, B, C2, accumulate=layout == hiplib.TN)
    assert torch.equal(C, C2)
    # linearity in A (exact in fp32 accumulation up to the final rounding): (2A) B == 2 (A B)
    C3 = torch.zeros_like(C)
    hiplib.gemm(layout, (A.float() * 2).to(A.dtype), B, C3, accumulate=layout == hiplib.TN)
    assert torch.equal(C3.float(), C.float() * 2)


@pytest.mark.parametrize("MB,HEADS", [(MB, HEADS), (MB5, HEADS5)], ids=["gpt2-medium", "gpt2-1.5b"])
@pytest.mark.parametrize("mask", ["causal", "key_padding"])
def test_attention_full_shape_properties(hiplib, mask, MB, HEADS):
    ROWS = MB * SEQ
    h = HEADS * 64
    qkv = randn(ROWS, 3 * h, seed=4, scale=0.7)
    out, lse = torch.empty(ROWS, h, dtype=torch.bfloat16, device=DEV), torch.empty(MB, HEADS, SEQ, device=DEV)
    lens = None
    if mask == "key_padding":
        lens = torch.randint(128, SEQ + 1, (MB,), generator=torch.Generator().manual_seed(5), dtype=torch.int32).to(DEV)
    code = hiplib.MASK_CODES[mask]
    hiplib.attention_fwd(qkv, out, lse, MB, HEADS, SEQ, code, lens)
    # oracle on two (batch, head) pairs
    for b, a in [(0, 0), (MB - 1, HEADS - 1)]:
        rows = slice(b * SEQ, (b + 1) * SEQ)
        q, k, v = [qkv[rows, i * h + a * 64: i * h + (a + 1) * 64].double().cpu() for i in range(3)]
        sc = q @ k.t() / 8.0
        if mask == "causal":
            sc = sc.masked_fill(~torch.tril(torch.ones(SEQ, SEQ, dtype=torch.bool)), -1e9)
        else:
            sc = sc.masked_fill(torch.arange(SEQ).view(1, -1) >= int(lens[b]), -1e9)
        assert l2(out[rows, a * 64:(a + 1) * 64], torch.softmax(sc, -1) @ v) < 1e-2
    # softmax rows sum to one: with V == 1 the context is exactly 1
    qkv1 = qkv.clone()
    qkv1[:, 2 * h:] = 1.0
    out1 = torch.empty_like(out)
    hiplib.attention_fwd(qkv1, out1, lse, MB, HEADS, SEQ, code, lens)
    assert float((out1.float() - 1).abs().max()) < 1e-2
    if mask == "causal":
        # causality: changing keys/values at positions >= 512 leaves the first 512 outputs bit-identical
        qkv2 = qkv.clone()
        view = qkv2.view(MB, SEQ, 3 * h)
        view[:, 512:, h:] = randn(MB, SEQ - 512, 2 * h, seed=6)
        out2 = torch.empty_like(out)
        hiplib.attention_fwd(qkv2, out2, lse, MB, HEADS, SEQ, code, lens)
        assert torch.equal(out.view(MB, SEQ, h)[:, :512], out2.view(MB, SEQ, h)[:, :512])
    # backward: reproducible, finite, and dV of fully masked keys is zero
    d_out = randn(ROWS, h, seed=7)
    hiplib.attention_fwd(qkv, out, lse, MB, HEADS, SEQ, code, lens)
    delta = torch.empty(MB, HEADS, SEQ, device=DEV)
    d1, d2 = torch.empty_like(qkv), torch.empty_like(qkv)
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d1, MB, HEADS, SEQ, code, lens)
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d2, MB, HEADS, SEQ, code, lens)
    assert torch.equal(d1, d2) and torch.isfinite(d1.float()).all()
    if mask == "key_padding":
        b = int(torch.argmin(lens))
        dead = d1.view(MB, SEQ, 3 * h)[b, int(lens[b]):, h:]
        assert float(dead.float().abs().max()) == 0.0


def test_attention_bert_large_shape_with_ragged_keys(hiplib):
    """The BERT-large stage's attention (16 samples of 512 positions, 16 heads, key lengths uniform in [128, 512]):
    forward and all three input gradients of the shortest and the longest sample against fp64 autograd, padded
    keys without probability mass or gradient, rows normalised."""
    mb, heads, seq = 16, 16, 512
    h = heads * 64
    rows = mb * seq
    qkv = randn(rows, 3 * h, seed=14, scale=0.7)
    lens = torch.randint(128, seq + 1, (mb,), generator=torch.Generator().manual_seed(15), dtype=torch.int32)
    lens[3], lens[11] = 128, 512
    lens_d = lens.to(DEV)
    code = hiplib.MASK_CODES["key_padding"]
    out, lse = torch.empty(rows, h, dtype=torch.bfloat16, device=DEV), torch.empty(mb, heads, seq, device=DEV)
    hiplib.attention_fwd(qkv, out, lse, mb, heads, seq, code, lens_d)
    d_out = randn(rows, h, seed=16)
    delta, d_qkv = torch.empty(mb, heads, seq, device=DEV), torch.empty_like(qkv)
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d_qkv, mb, heads, seq, code, lens_d)
    for b, a in [(3, 0), (11, heads - 1), (7, 5)]:
        rs = slice(b * seq, (b + 1) * seq)
        q, k, v = [qkv[rs, i * h + a * 64: i * h + (a + 1) * 64].double().cpu().requires_grad_(True) for i in range(3)]
        sc = (q @ k.t() / 8.0).masked_fill(torch.arange(seq).view(1, -1) >= int(lens[b]), -1e9)
        ctx = torch.softmax(sc, -1) @ v
        ctx.backward(d_out[rs, a * 64:(a + 1) * 64].double().cpu())
        assert l2(out[rs, a * 64:(a + 1) * 64], ctx.detach()) < 1e-2
        for i, t in enumerate((q, k, v)):
            assert l2(d_qkv[rs, i * h + a * 64: i * h + (a + 1) * 64], t.grad) < 2e-2, (b, a, i)
    dead = d_qkv.view(mb, seq, 3 * h)[3, 128:, h:]
    assert float(dead.float().abs().max()) == 0.0
    qkv1 = qkv.clone()
    qkv1[:, 2 * h:] = 1.0
    hiplib.attention_fwd(qkv1, out, lse, mb, heads, seq, code, lens_d)
    assert float((out.float() - 1).abs().max()) < 1e-2


@pytest.mark.parametrize("MB,HID,HEADS,FFN", [(MB, HID, HEADS, FFN), (MB5, HID5, HEADS5, FFN5)], ids=["gpt2-medium", "gpt2-1.5b"])
def test_rc_bit_exact_full_layer(hiplib, MB, HID, HEADS, FFN):
    """One own + one shadow layer at the benchmark's layer shape: the redundant forward equals a normal
    forward of the same layer bit for bit, on either stream arrangement."""
    variant = dict(activation="gelu_tanh", ln="standard", mask="causal")
    M = 2
    outs = []
    for rc_stream in (False, True):
        specs = [LayerSpec(TransformerLayer, HID, HEADS, FFN, **variant) for _ in range(4)]
        model = PipelineModule(specs, num_stages=4, partition_method="uniform", stage_id=1, dtype=torch.bfloat16, device=DEV)
        q = SeededActivationQueue((MB, SEQ, HID), torch.bfloat16, M, stage_ids=[1, 2], seed=11, device=DEV)
        cfg = {"train_micro_batch_size_per_gpu": MB, "gradient_accumulation_steps": M, "bf16": {"enabled": True}}
        engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                                activation_queue=q, rc_stream=rc_stream, install_signal_handler=False)
        keep = {}
        engine._clean_pipe_buffers = lambda: keep.update({k: [None if t is None else t.clone() for t in v]
                                                          for k, v in engine.pipe_buffers.items()})
        engine.train_batch()
        torch.cuda.synchronize()
        outs.append(keep)
        del engine
    model2 = PipelineModule([LayerSpec(TransformerLayer, HID, HEADS, FFN, **variant) for _ in range(4)], num_stages=4,
                            partition_method="uniform", stage_id=2, dtype=torch.bfloat16, device=DEV)
    ctx2 = model2.prepare_context([2], MB, SEQ)
    model2.allocate_stash(2, ctx2, 1)
    for k in range(M):
        normal = model2.forward(outs[0]["output_1"][k], 2, slot=0, ctx=ctx2)
        torch.cuda.synchronize()
        assert torch.equal(normal, outs[0]["output_2"][k])
        assert torch.equal(outs[0]["output_2"][k], outs[1]["output_2"][k])
        assert torch.equal(outs[0]["input_grad_1"][k], outs[1]["input_grad_1"][k])


def test_adam_full_stage_arena(hiplib):
    """75.6 M parameters (six layers) in one launch; the first and last million elements bit-exact with the oracle."""
    n = 6 * 12596224
    g = torch.Generator(device=DEV).manual_seed(8)
    P = torch.randn(n, generator=g, device=DEV)
    G = torch.randn(n, generator=g, device=DEV)
    Mo, V = torch.zeros(n, device=DEV), torch.zeros(n, device=DEV)
    LP = torch.empty(n, dtype=torch.bfloat16, device=DEV)
    p0, g0 = P.clone(), G.clone()
    hiplib.adam_multi([G], [P], [Mo], [V], [LP], lr=1e-3, beta1=0.9, beta2=0.999, eps=1e-8, step=1, zero_grad=True)
    for sl in (slice(0, 1 << 20), slice(n - (1 << 20), n)):
        p = p0[sl].cpu().numpy().copy()
        m, v = np.zeros_like(p), np.zeros_like(p)
        oadam.adam_step(p, g0[sl].cpu().numpy(), m, v, 1)
        assert np.array_equal(P[sl].cpu().numpy(), p) and np.array_equal(V[sl].cpu().numpy(), v)
    assert torch.equal(LP, P.to(torch.bfloat16)) and float(G.abs().max()) == 0.0
    # first step with zero moments moves every parameter by lr * g/(|g| + eps') ~ lr
    assert float((P - p0).abs().max()) <= 1.001e-3


def test_failover_at_the_gpt2_1p5b_layer_shape(hiplib):
    """One own and one shadow layer of the GPT-2-1.5B stage (hidden 1600, 25 heads, ffn 6400, seq 1024,
    micro-batch 4), two micro-batches, the successor preempted at the second: the promoted layer's backward runs
    from the stashed redundant forward for micro-batch 0 and after a normal forward for micro-batch 1.  Gradients
    of both stages and the loss against the CPU oracle (fp32 arithmetic on the engine's bf16 weights), 2e-2."""
    from oracle.stage import OraclePeer, OracleStage
    variant = dict(activation="gelu_tanh", ln="standard", mask="causal")
    S, sid, M = 4, 1, 2
    specs = [LayerSpec(TransformerLayer, HID5, HEADS5, FFN5, **variant) for _ in range(S)]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=torch.bfloat16, device=DEV)
    q = SeededActivationQueue((MB5, SEQ, HID5), torch.bfloat16, M, stage_ids=[sid, sid + 1], seed=13, grad_mode="mse", device=DEV)
    cfg = {"train_micro_batch_size_per_gpu": MB5, "gradient_accumulation_steps": M, "bf16": {"enabled": True}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                            activation_queue=q, install_signal_handler=False)
    st = OracleStage(ol.TransformerCfg(hidden=HID5, heads=HEADS5, ffn=FFN5, **variant), list(range(S + 1)), sid, M,
                     dtype=torch.float32, redundancy_level=1, eager=True)
    for s_ in list(st.params):
        sp = engine.module.stage_params[s_]
        named = sp.named(sp.compute)
        for key, t in st.named_params(s_).items():
            with torch.no_grad():
                t.copy_(named[key].float().cpu())
    acts = [a.float().cpu() for a in q.activations]
    targets = [t.float().cpu() for t in q.targets[sid + 1]]
    true_grads = []
    for k in range(M):
        o1 = st.forward(acts[k], sid).detach().requires_grad_(True)
        (torch.nn.functional.mse_loss(st.forward(o1, sid + 1), targets[k]) / M).backward()
        true_grads.append(o1.grad)
    for layers in st.params.values():
        for p in layers:
            for t in p.values():
                t.grad = None
    peer = OraclePeer(acts, M, grads={sid: true_grads}, targets={sid + 1: targets})
    peer.dead_from, peer.dead_stage = 1, sid
    st.run_batch(peer, optimizer_step=False)

    q.set_grads(sid, [g.view(MB5, SEQ, HID5) for g in true_grads])
    q.targets.pop(sid)                      # own outputs go to a live successor, not to a loss head
    orig_send = q.send_activation
    q.send_activation = lambda k, t, stage_id, stream=None: (q._check_alive(k, stage_id) if stage_id == sid
                                                              else orig_send(k, t, stage_id, stream=stream))
    q.preempt_successor(1, sid)
    from bamboo_amd import schedule
    engine._INSTRUCTION_MAP = dict(engine._INSTRUCTION_MAP)
    engine._INSTRUCTION_MAP[schedule.OptimizerStep] = lambda self_: None
    loss = engine.train_batch()
    torch.cuda.synchronize()
    assert engine.stage_ids == [sid, sid + 1]
    for s_ in (sid, sid + 1):
        ref = st.named_grads(s_)
        floor = 1e-3 * max(float(g.abs().max()) for g in ref.values())
        for name, g in engine.module.get_named_grad(s_):
            r = ref[name].double()
            err = float((g.double().cpu() - r).norm() / r.norm().clamp_min(floor * r.numel() ** 0.5))
            assert err < 2e-2, (s_, name, err)
    assert abs(float(loss) - float(peer.loss) / M) < 2e-2 * float(peer.loss) / M


# ---------------------------------------------------------------- GPT-2-small stage (fp32) at its own shapes
MB1, SEQ1, HID1, HEADS1, FFN1 = 4, 512, 768, 12, 3072


def test_gpt2_small_stage_full_shape_fp32_matches_oracle(hiplib):
    """The fp32 configuration at its own sizes (hidden 768, 12 heads, ffn 3072, seq 512, micro-batch 4, causal,
    MSE to seeded N(0,1) targets): one own and one shadow layer, two micro-batches, redundant forwards on; stage
    outputs (own and redundant) within 1e-5 and every gradient within 1e-4 of the fp64 CPU oracle, largest error
    over the tensor's largest magnitude.  This is the only place where the fp32 path -- `gemm_f32_kernel` with
    K = 768 / 3072 and the unfused attention (batched head products + softmax over 4 x 12 x 512 x 512
    probabilities) -- meets the oracle at the sizes it is benchmarked on."""
    from tests.test_gpu_stage import GPT_VARIANT, NoStep, build, grad_floor, oracle_for, rel_err
    L, S, sid, M = 1, 4, 1, 2
    engine, q = build(HID1, HEADS1, FFN1, L, S, sid, MB1, M, SEQ1, torch.float32, GPT_VARIANT, 1, True, grad_mode="mse")
    assert not engine.module.func_buckets[sid][0].fused_attention(engine.ctx)
    st, peer = oracle_for(engine, q, GPT_VARIANT, HID1, HEADS1, FFN1, L, S, sid, M, 1, True)
    keep = {}
    with NoStep(engine):
        engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
        loss = engine.train_batch()
    torch.cuda.synchronize()
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    rel_err.lowp = False
    rows = MB1 * SEQ1
    for k in range(M):
        assert rel_err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().view(rows, HID1)) < 1e-5, k
        assert rel_err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().view(rows, HID1)) < 1e-5, k
        assert rel_err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].view(rows, HID1)) < 1e-4, k
    ref = st.named_grads(sid)
    for name, g in engine.module.get_named_grad(sid):
        assert rel_err(g, ref[name], grad_floor(ref)) < 1e-4, name
    assert abs(float(loss) - float(peer.loss) / M) < 1e-5 * float(peer.loss) / M


@pytest.mark.parametrize("mask", ["causal", "key_padding"])
def test_unfused_attention_fp32_at_12_heads_512_positions(hiplib, mask):
    """The fp32 attention core by itself at the GPT-2-small stage's size (4 x 12 heads x 512 positions, head
    dimension 64): scores, masked softmax, context and the three input gradients against fp64 autograd on
    ``softmax(Q K^T / sqrt(d) [masked]) V``, 1e-5 forward / 1e-4 backward of each tensor's largest magnitude."""
    from bamboo_amd.layers import StageContext
    b, a, s, d = MB1, HEADS1, SEQ1, 64
    h = a * d
    layer = TransformerLayer(h, a, 4 * h, activation="gelu_tanh", ln="standard", mask=mask)
    ctx = StageContext(b, s, torch.float32, torch.device(DEV))
    lens = None
    if mask == "key_padding":
        lens = torch.randint(128, s + 1, (b,), generator=torch.Generator().manual_seed(8), dtype=torch.int32).to(DEV)
        lens[0] = s
    ctx.key_len = lens
    qkv = randn(b * s, 3 * h, seed=41, scale=0.7, dtype=torch.float32)
    d_ctx = randn(b * s, h, seed=42, dtype=torch.float32)
    st = {"qkv": qkv, "ctx": torch.empty(b * s, h, device=DEV), "prob": torch.empty(b, a, s, s, device=DEV)}
    ctx.ensure_scratch([("d_prob", (b, a, s, s), torch.float32)])
    assert not layer.fused_attention(ctx)
    layer._attention_fwd(st, ctx)
    d_qkv = torch.empty_like(qkv)
    layer._attention_bwd(d_ctx, d_qkv, st, ctx)
    torch.cuda.synchronize()
    # fp64 autograd on the CPU
    x = qkv.double().cpu().requires_grad_(True)
    qq, kk, vv = [x[:, i * h:(i + 1) * h].view(b, s, a, d).transpose(1, 2) for i in range(3)]
    scores = qq @ kk.transpose(-2, -1) / math.sqrt(d)
    if mask == "causal":
        keep_ = torch.tril(torch.ones(s, s, dtype=torch.bool)).view(1, 1, s, s)
    else:
        keep_ = torch.arange(s).view(1, 1, 1, s) < lens.cpu().view(b, 1, 1, 1)
    prob = torch.softmax(scores.masked_fill(~keep_, -1e9), dim=-1)
    out = (prob @ vv).transpose(1, 2).reshape(b * s, h)
    out.backward(d_ctx.double().cpu())
    err = lambda got, want: float((got.double().cpu() - want).abs().max() / want.abs().max())
    assert err(st["prob"], prob.detach()) < 1e-5
    assert err(st["ctx"], out.detach()) < 1e-5
    for i, name in enumerate("qkv"):
        assert err(d_qkv[:, i * h:(i + 1) * h], x.grad[:, i * h:(i + 1) * h]) < 1e-4, f"d{name}"


@pytest.mark.parametrize("mask", ["none", "causal", "key_padding"])
@pytest.mark.parametrize("d,a,fused", [(32, 4, True), (32, 3, False), (128, 4, True), (96, 2, False)],
                         ids=["d32-pairs-fused", "d32-odd-heads", "d128-fused", "d96"])
def test_bf16_attention_with_other_head_widths(hiplib, mask, d, a, fused):
    """bf16 heads that are not 64 wide, through the layer's attention calls.  An even number of 32-wide heads (the
    reference's GPT-2 script defaults to 512 / 16 = 32, gpt2.py:212-214) runs on the fused kernels, which take the
    heads in pairs, and so do 128-wide heads (two column panels); an odd number of 32-wide heads and other widths take
    the path that materialises the probabilities.
    Context and the three input gradients against fp64 autograd on ``softmax(Q K^T / sqrt(d) [masked]) V``, 2e-2 of
    each tensor's largest magnitude, for the three masks."""
    from bamboo_amd.layers import StageContext
    b, s = 2, 256
    h = a * d
    layer = TransformerLayer(h, a, 4 * h, activation="gelu_tanh", ln="standard", mask=mask)
    ctx = StageContext(b, s, torch.bfloat16, torch.device(DEV))
    lens = None
    if mask == "key_padding":
        lens = torch.tensor([s, 77], dtype=torch.int32, device=DEV)
    ctx.key_len = lens
    qkv = randn(b * s, 3 * h, seed=51, scale=0.7)
    d_ctx = randn(b * s, h, seed=52)
    st = {"qkv": qkv, "ctx": torch.empty(b * s, h, dtype=torch.bfloat16, device=DEV),
          "prob": torch.empty(b, a, s, s, dtype=torch.bfloat16, device=DEV), "lse": torch.empty(b, a, s, device=DEV)}
    ctx.ensure_scratch([("d_prob", (b, a, s, s), torch.bfloat16), ("attn_delta", (b, a, s), torch.float32)])
    assert layer.fused_attention(ctx) == fused
    layer._attention_fwd(st, ctx)
    d_qkv = torch.empty_like(qkv)
    layer._attention_bwd(d_ctx, d_qkv, st, ctx)
    torch.cuda.synchronize()
    x = qkv.double().cpu().requires_grad_(True)
    qq, kk, vv = [x[:, i * h:(i + 1) * h].view(b, s, a, d).transpose(1, 2) for i in range(3)]
    scores = qq @ kk.transpose(-2, -1) / math.sqrt(d)
    if mask == "causal":
        scores = scores.masked_fill(~torch.tril(torch.ones(s, s, dtype=torch.bool)).view(1, 1, s, s), -1e9)
    elif mask == "key_padding":
        scores = scores.masked_fill(~(torch.arange(s).view(1, 1, 1, s) < lens.cpu().view(b, 1, 1, 1)), -1e9)
    out = (torch.softmax(scores, dim=-1) @ vv).transpose(1, 2).reshape(b * s, h)
    out.backward(d_ctx.double().cpu())
    err = lambda got, want: float((got.double().cpu() - want).abs().max() / want.abs().max())
    assert err(st["ctx"], out.detach()) < 2e-2
    for i, name in enumerate("qkv"):
        assert err(d_qkv[:, i * h:(i + 1) * h], x.grad[:, i * h:(i + 1) * h]) < 2e-2, f"d{name}"
