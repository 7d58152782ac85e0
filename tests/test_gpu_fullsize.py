"""Checks at the full shapes of the benchmark configuration (GPT-2-medium stage: rows 8192, hidden 1024,
ffn 4096, 16 heads, seq 1024) through properties that do not need a full CPU run: bit-reproducibility,
oracle values on sampled rows / heads, softmax normalisation, causality, RC bit-exactness."""
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


def randn(*shape, seed=0, scale=1.0, dtype=torch.bfloat16):
    g = torch.Generator(device=DEV).manual_seed(seed)
    return (torch.randn(*shape, generator=g, device=DEV) * scale).to(dtype)


def l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("layout,M,N,K", [(0, ROWS, FFN, HID), (0, ROWS, 3 * HID, HID), (0, ROWS, HID, FFN),
                                          (1, ROWS, HID, FFN), (1, ROWS, FFN, HID), (2, FFN, HID, ROWS), (2, HID, HID, ROWS)])
def test_gemm_full_shapes_sampled(hiplib, layout, M, N, K):
    a_shape = (K, M) if layout == hiplib.TN else (M, K)
    b_shape = (N, K) if layout == hiplib.NT else (K, N)
    A, B = randn(*a_shape, seed=1), randn(*b_shape, seed=2, scale=0.05)
    C = torch.empty(M, N, dtype=torch.float32 if layout == hiplib.TN else torch.bfloat16, device=DEV)
    if layout == hiplib.TN:
        C.zero_()
    hiplib.gemm(layout, A, B, C, accumulate=layout == hiplib.TN)
    idx = torch.randint(0, M, (48,), generator=torch.Generator().manual_seed(3)).to(DEV)
    Ar = (A[:, idx].t() if layout == hiplib.TN else A[idx]).double()
    ref = Ar @ (B.double().t() if layout == hiplib.NT else B.double())
    assert l2(C[idx], ref) < 1e-2
    C2 = torch.zeros_like(C)
    hiplib.gemm(layout, A, B, C2, accumulate=layout == hiplib.TN)
    assert torch.equal(C, C2)
    # linearity in A (exact in fp32 accumulation up to the final rounding): (2A) B == 2 (A B)
    C3 = torch.zeros_like(C)
    hiplib.gemm(layout, (A.float() * 2).to(A.dtype), B, C3, accumulate=layout == hiplib.TN)
    assert torch.equal(C3.float(), C.float() * 2)


@pytest.mark.parametrize("mask", ["causal", "key_padding"])
def test_attention_full_shape_properties(hiplib, mask):
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


def test_rc_bit_exact_full_layer(hiplib):
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
