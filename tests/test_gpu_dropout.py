"""Dropout on the GPU: the generic kernel, the GEMM epilogues and the fused attention kernels against references
built from the oracle's explicit masks; stage-level parity and the bit-exactness of redundant forwards at p = 0.1."""
import math

import numpy as np
import pytest
import torch

import bamboo_amd
from bamboo_amd import LayerSpec, PipelineModule, SeededActivationQueue, TransformerLayer
from oracle import dropout as od
from oracle import layers as ol
from oracle.stage import OraclePeer, OracleStage

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
KEY = od.key(1234, 3, 2, 7, 1)


def l2(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).norm() / b.norm())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_dropout_kernel_makes_the_oracle_decisions(hiplib, dtype):
    n, p = 8 * 12345, 0.1
    x = (torch.randn(n, device=DEV) + 3).to(dtype)        # no zeros: the mask can be read off the result
    y = torch.empty_like(x)
    hiplib.dropout_apply(x, y, p, KEY)
    m = torch.from_numpy(od.mask(p, KEY, (n,))).to(DEV)
    assert torch.equal(y != 0, m.bool())
    want = (x.float() * (1.0 / (1.0 - np.float32(p)))).to(dtype)
    assert torch.equal(y[m.bool()], want[m.bool()])
    hiplib.dropout_apply(x, x, p, KEY)                     # in place
    assert torch.equal(x, y)
    z = torch.empty_like(x)
    hiplib.dropout_apply(y, z, 0.0, KEY)                   # p = 0: a copy
    assert torch.equal(z, y)


@pytest.mark.parametrize("dtype,M,N,K", [(torch.bfloat16, 512, 384, 256), (torch.bfloat16, 200, 72, 96), (torch.float32, 130, 68, 40),
                                         (torch.bfloat16, 7168, 4096, 576)],
                         ids=["bf16-dma", "bf16-fallback", "fp32", "bf16-persistent"])
@pytest.mark.parametrize("epi", ["none", "act", "act_dact", "residual"])
def test_gemm_epilogue_dropout(hiplib, dtype, M, N, K, epi):
    p = 0.25
    g = torch.Generator(device=DEV).manual_seed(5)
    A = (torch.randn(M, K, generator=g, device=DEV) * 0.5).to(dtype)
    B = (torch.randn(N, K, generator=g, device=DEV) * 0.5).to(dtype)
    bias = torch.randn(N, generator=g, device=DEV).to(dtype)
    resid = torch.randn(M, N, generator=g, device=DEV).to(dtype)
    C, aux = torch.empty(M, N, dtype=dtype, device=DEV), torch.empty(M, N, dtype=dtype, device=DEV)
    kw = dict(bias=bias, dropout=(p, KEY))
    if epi == "act":
        kw.update(epilogue=hiplib.EPI_ACT, act=hiplib.ACT_GELU_TANH)
    elif epi == "act_dact":
        kw.update(epilogue=hiplib.EPI_ACT_DACT, act=hiplib.ACT_GELU_TANH, aux_out=aux)
    elif epi == "residual":
        kw.update(epilogue=hiplib.EPI_RESIDUAL, resid=resid)
    hiplib.gemm(hiplib.NT, A, B, C, **kw)
    m = torch.from_numpy(od.mask(p, KEY, (M, N))).to(DEV)
    u = (A.double() @ B.double().t() + bias.double())
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    if epi in ("act", "act_dact"):
        ug = u.clone().requires_grad_(True)
        act = torch.nn.functional.gelu(ug, approximate="tanh")
        (dact,) = torch.autograd.grad(act.sum(), ug)
        assert l2(C, act.detach() * m / (1 - p)) < tol
        if epi == "act_dact":
            assert l2(aux, dact * m / (1 - p)) < tol
            assert float(aux[m == 0].abs().max()) == 0.0          # the derivative is dropped where the activation is
    elif epi == "residual":
        assert l2(C, u * m / (1 - p) + resid.double()) < tol
    else:
        assert l2(C, u * m / (1 - p)) < tol
        assert torch.equal(C == 0, m == 0) or float(((C == 0) != (m == 0)).float().mean()) < 1e-3
    # same key, same decisions, same bits
    C2 = torch.empty_like(C)
    hiplib.gemm(hiplib.NT, A, B, C2, **{**kw, **({"aux_out": torch.empty_like(aux)} if epi == "act_dact" else {})})
    assert torch.equal(C, C2)


@pytest.mark.parametrize("mask", ["none", "causal", "key_padding"])
@pytest.mark.parametrize("batch,heads,seq,d", [(2, 2, 128, 64), (1, 3, 200, 64), (2, 4, 128, 32), (1, 2, 200, 32), (2, 2, 128, 128),
                                               (1, 1, 200, 128)])
def test_fused_attention_dropout_fwd_bwd(hiplib, mask, batch, heads, seq, d):
    """softmax(QK^T / sqrt(d), mask) -> dropout -> V with the oracle's explicit mask through torch autograd in fp64,
    against the fused kernels that evaluate the decisions themselves: context, dQ, dK, dV (64-wide heads, and 32-wide
    heads in pairs: every head keeps its own decisions)."""
    p, h = 0.2, heads * d
    g = torch.Generator(device=DEV).manual_seed(9)
    qkv = (torch.randn(batch * seq, 3 * h, generator=g, device=DEV) * 0.7).to(torch.bfloat16)
    d_out = torch.randn(batch * seq, h, generator=g, device=DEV).to(torch.bfloat16)
    lens = None
    if mask == "key_padding":
        lens = torch.tensor([seq - 37, seq][:batch] if batch > 1 else [seq - 37], dtype=torch.int32, device=DEV)
    code = hiplib.MASK_CODES[mask]
    out, lse = torch.empty(batch * seq, h, dtype=torch.bfloat16, device=DEV), torch.empty(batch, heads, seq, device=DEV)
    hiplib.attention_fwd(qkv, out, lse, batch, heads, seq, code, lens, dropout=(p, KEY))
    delta, d_qkv = torch.empty(batch, heads, seq, device=DEV), torch.empty_like(qkv)
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d_qkv, batch, heads, seq, code, lens, dropout=(p, KEY))
    # reference
    x = qkv.double().cpu().view(batch, seq, 3, heads, d).requires_grad_(True)
    q, k, v = [x[:, :, i].transpose(1, 2) for i in range(3)]
    sc = q @ k.transpose(-2, -1) / d ** 0.5
    if mask == "causal":
        sc = sc.masked_fill(~torch.tril(torch.ones(seq, seq, dtype=torch.bool)), -1e9)
    elif mask == "key_padding":
        sc = sc.masked_fill(torch.arange(seq).view(1, 1, 1, seq) >= lens.cpu().view(batch, 1, 1, 1), -1e9)
    m = torch.from_numpy(od.mask(p, KEY, (batch, heads, seq, seq)))
    ctx = ((sc.softmax(-1) * m / (1 - p)) @ v).transpose(1, 2).reshape(batch * seq, h)
    ctx.backward(d_out.double().cpu())
    assert l2(out, ctx.detach()) < 1.5e-2
    ref = x.grad.view(batch * seq, 3 * h)
    for i, name in enumerate(("dq", "dk", "dv")):
        assert l2(d_qkv[:, i * h:(i + 1) * h], ref[:, i * h:(i + 1) * h]) < 2e-2, name
    # without dropout the kernels give something else; with it, twice the same bits
    out0 = torch.empty_like(out)
    hiplib.attention_fwd(qkv, out0, lse, batch, heads, seq, code, lens)
    assert not torch.equal(out0, out)
    out2 = torch.empty_like(out)
    hiplib.attention_fwd(qkv, out2, lse, batch, heads, seq, code, lens, dropout=(p, KEY))
    assert torch.equal(out2, out)


def build(dtype, rl, eager, p, rc_stream=False, seed=7, M=4):
    hid, heads, ffn, L, S, sid, mb, seq = 128, 2, 256, 2, 4, 1, 2, 64
    variant = dict(activation="gelu_tanh", ln="standard", mask="causal", dropout=p)
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **variant) for _ in range(L * S)]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV, base_seed=4321)
    q = SeededActivationQueue((mb, seq, hid), dtype, M, stage_ids=[sid, sid + 1], seed=seed, device=DEV)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M,
           "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=rl, eager_recovery=eager,
                                            activation_queue=q, rc_stream=rc_stream, install_signal_handler=False)
    return engine, q, (hid, heads, ffn, L, S, sid, mb, seq, variant)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_stage_with_dropout_matches_oracle(hiplib, dtype):
    """Own forward + backward and the redundant forwards at p = 0.1 (fp32: unfused attention with the dropout kernel,
    bf16: fused) against the oracle stage that builds the same masks from (base seed, batch counter, micro-batch,
    layer, site); second batch after an optimizer step (the batch counter moves the masks)."""
    p, M = 0.1, 4
    engine, q, (hid, heads, ffn, L, S, sid, mb, seq, variant) = build(dtype, 1, True, p)
    cfg = ol.TransformerCfg(hidden=hid, heads=heads, ffn=ffn, **variant)
    st = OracleStage(cfg, [i * L for i in range(S + 1)], sid, M, base_seed=4321, dtype=torch.float64, redundancy_level=1, eager=True)
    for s_ in list(st.params):
        sp = engine.module.stage_params[s_]
        named = sp.named(sp.compute)
        for key, t in st.named_params(s_).items():
            with torch.no_grad():
                t.copy_(named[key].double().cpu())
    peer = OraclePeer([a.double().cpu() for a in q.activations], M, grads={s_: [g.double().cpu() for g in gs] for s_, gs in q.grads.items()})
    keep = {}
    from bamboo_amd import schedule
    engine._INSTRUCTION_MAP = dict(engine._INSTRUCTION_MAP)
    engine._INSTRUCTION_MAP[schedule.OptimizerStep] = lambda self_: None
    engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
    engine.train_batch()
    torch.cuda.synchronize()
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    ta, tg = (1e-5, 1e-4) if dtype == torch.float32 else (2e-2, 2e-2)
    lowp = dtype == torch.bfloat16
    err = lambda a, b: l2(a, b) if lowp else float((a.double().cpu() - b.double().cpu()).abs().max() / b.abs().max())
    for k in range(M):
        assert err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().view(mb * seq, hid)) < ta
        assert err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().view(mb * seq, hid)) < ta
        assert err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].view(mb * seq, hid)) < tg
    ref = st.named_grads(sid)
    floor = 1e-3 * max(float(g.abs().max()) for g in ref.values())
    for name, gr in engine.module.get_named_grad(sid):
        r = ref[name]
        e = float((gr.double().cpu() - r).norm() / r.norm().clamp_min(floor * r.numel() ** 0.5)) if lowp else \
            float((gr.double().cpu() - r).abs().max() / max(float(r.abs().max()), floor))
        assert e < tg, name
    # dropout really happened: the same engine with p = 0 gives other outputs
    e0, _, _ = build(dtype, 0, False, 0.0)
    keep0 = {}
    e0._clean_pipe_buffers = lambda: keep0.update({k: list(v) for k, v in e0.pipe_buffers.items()})
    e0.train_batch()
    assert not torch.equal(keep0[f"output_{sid}"][0], keep[f"output_{sid}"][0])


@pytest.mark.parametrize("rc_stream", [False, True], ids=["one-stream", "rc-stream"])
def test_rc_bit_exact_with_dropout(hiplib, rc_stream):
    """p = 0.1: the redundant forward of the shadow layers equals a normal forward of the same layers on the same
    input bit for bit (the decisions depend on the micro-batch, the layer and the batch counter, not on who runs the
    forward) and RC changes nothing in the own results, over two batches with an optimizer step between them."""
    p, M = 0.1, 4
    dtype = torch.bfloat16
    runs = {}
    for tag, (rl, eager) in {"off": (0, False), "on": (1, True)}.items():
        engine, q, meta = build(dtype, rl, eager, p, rc_stream=rc_stream and eager)
        keep = {}

        def snapshot_then_clean(keep=keep, engine=engine, clean=engine._clean_pipe_buffers):
            keep.update({k: [None if t is None else t.clone() for t in v] for k, v in engine.pipe_buffers.items()})
            clean()
        engine._clean_pipe_buffers = snapshot_then_clean
        losses = [float(engine.train_batch()) for _ in range(2)]     # two batches: the counter moves the masks
        torch.cuda.synchronize()
        runs[tag] = (engine, keep, losses)
    hid, heads, ffn, L, S, sid, mb, seq, variant = meta
    for k in range(M):
        assert torch.equal(runs["off"][1][f"output_{sid}"][k], runs["on"][1][f"output_{sid}"][k])
        assert torch.equal(runs["off"][1][f"input_grad_{sid}"][k], runs["on"][1][f"input_grad_{sid}"][k])
    a, b = runs["off"][0].module.stage_params[sid], runs["on"][0].module.stage_params[sid]
    assert torch.equal(a.master, b.master)
    # a stage of its own that runs the shadow layers normally, in the second batch (batch counter 1)
    engine, keep, _ = runs["on"]
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **variant) for _ in range(L * S)]
    model2 = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid + 1, dtype=dtype, device=DEV, base_seed=4321)
    ctx2 = model2.prepare_context([sid + 1], mb, seq)
    model2.allocate_stash(sid + 1, ctx2, 1)
    for k in range(M):
        ctx2.dropout_base = (4321, 1, k)
        normal = model2.forward(keep[f"output_{sid}"][k], sid + 1, slot=0, ctx=ctx2)
        torch.cuda.synchronize()
        assert torch.equal(normal, keep[f"output_{sid + 1}"][k]), f"micro-batch {k}"
    ctx2.dropout_base = (4321, 0, 0)     # another batch counter: other masks
    other = model2.forward(keep[f"output_{sid}"][0], sid + 1, slot=0, ctx=ctx2)
    assert not torch.equal(other, keep[f"output_{sid + 1}"][0])
    with pytest.raises(bamboo_amd.PipelineError, match="dropout"):
        side = torch.cuda.Stream()
        with torch.cuda.stream(side):
            specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **variant) for _ in range(L * S)]
            m3 = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
            q3 = SeededActivationQueue((mb, seq, hid), dtype, M, stage_ids=[sid], device=DEV)
            bamboo_amd.initialize(model=m3, config={"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M,
                                                    "bf16": {"enabled": True}}, activation_queue=q3, use_graphs=True,
                                  install_signal_handler=False)


def test_dropout_indices_past_32_bits(hiplib):
    """Tensors of 2^32 elements and more take the 64-bit index arithmetic (smaller ones, i.e. every other test, the
    32-bit one): the stand-alone kernel over 2^32 + 4096 elements and the epilogue of a 65536 x 65544 product, on
    sampled elements either side of the 2^32 boundary, against the oracle's decisions."""
    p = 0.25
    n = (1 << 32) + 4096
    x = torch.ones(n, dtype=torch.bfloat16, device=DEV)
    y = torch.empty_like(x)
    hiplib.dropout_apply(x, y, p, KEY)
    rng = np.random.default_rng(8)
    idx = np.concatenate([np.arange(64), (1 << 32) - 64 + np.arange(128), n - 64 + np.arange(64),
                          rng.integers(0, n, 4096)]).astype(np.int64)
    got = y[torch.from_numpy(idx).to(DEV)].float().cpu().numpy() != 0
    assert np.array_equal(got, od.keep(p, KEY, idx.astype(np.uint64)))
    assert abs(float((y[: 1 << 24] != 0).float().mean()) - (1 - p)) < 1e-3 and abs(float((y[-(1 << 24):] != 0).float().mean()) - (1 - p)) < 1e-3
    del x, y
    M, N, K = 65536, 65544, 64
    A = torch.full((M, K), 0.125, dtype=torch.bfloat16, device=DEV)
    B = torch.full((N, K), 0.125, dtype=torch.bfloat16, device=DEV)
    C = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)           # every element 1 before dropout
    hiplib.gemm(hiplib.NT, A, B, C, dropout=(p, KEY))
    ms = np.concatenate([[0, 1, M - 1, 65527, 65528], rng.integers(0, M, 512)]).astype(np.int64)
    ns = np.concatenate([[0, 7, N - 1, 8, 65543], rng.integers(0, N, 512)]).astype(np.int64)
    flat = ms * N + ns
    assert flat.max() >= 1 << 32
    got = C[torch.from_numpy(ms).to(DEV), torch.from_numpy(ns).to(DEV)].float().cpu().numpy()
    keep = od.keep(p, KEY, flat.astype(np.uint64))
    assert np.array_equal(got != 0, keep)
    assert np.allclose(got[keep], float(torch.tensor(1.0 / (1.0 - np.float32(p))).bfloat16()))


def test_attention_dropout_past_32_bits_of_probabilities(hiplib):
    """One head over 65536 positions: 2^32 probabilities, so the three fused kernels take the 64-bit index arithmetic.
    Sampled query rows of the context and of dQ, sampled key rows of dK and dV, against fp64 restatements built from
    the oracle's decisions."""
    p, s, d = 0.25, 65536, 64
    g = torch.Generator(device=DEV).manual_seed(21)
    qkv = (torch.randn(s, 3 * d, generator=g, device=DEV) * 0.5).bfloat16()
    d_out = torch.randn(s, d, generator=g, device=DEV).bfloat16()
    out, lse = torch.empty(s, d, dtype=torch.bfloat16, device=DEV), torch.empty(1, 1, s, device=DEV)
    delta, d_qkv = torch.empty(1, 1, s, device=DEV), torch.empty_like(qkv)
    code = hiplib.MASK_CODES["none"]
    hiplib.attention_fwd(qkv, out, lse, 1, 1, s, code, dropout=(p, KEY))
    hiplib.attention_bwd(qkv, out, d_out, lse, delta, d_qkv, 1, 1, s, code, dropout=(p, KEY))
    torch.cuda.synchronize()
    Q, K, V = [qkv[:, i * d:(i + 1) * d].double().cpu() for i in range(3)]
    dO, O = d_out.double().cpu(), out.double().cpu()
    scale = 1.0 / (1.0 - p)
    cols = torch.arange(s, dtype=torch.int64)
    for q in (0, 1, 40001, s - 1):
        sc = (K @ Q[q]) / 8.0
        prob = torch.softmax(sc, 0)
        keep = torch.from_numpy(od.keep(p, KEY, (q * s + cols.numpy()).astype(np.uint64))).double()
        pk = prob * keep * scale
        assert l2(out[q], pk @ V) < 1e-2, q
        dpk = (V @ dO[q]) * keep * scale                 # gradient of the kept-and-scaled probabilities
        dlt = float((dO[q] * O[q]).sum())                # rowsum(dO o O) = sum_kv P~ dP (what the kernels subtract)
        ds = prob * (dpk - dlt)
        assert l2(d_qkv[q, :d], (ds @ K) / 8.0) < 3e-2, q
    # full-column checks need every row's normaliser: recompute it in fp64 for all rows, blockwise
    lse64 = torch.empty(s, dtype=torch.float64)
    for lo in range(0, s, 4096):
        lse64[lo:lo + 4096] = torch.logsumexp((Q[lo:lo + 4096] @ K.t()) / 8.0, dim=1)
    dlt_all = (dO * O).sum(1)
    rows = torch.arange(s, dtype=torch.int64).numpy()
    for kv in (0, 3, 33333, s - 1):
        prob = torch.exp((Q @ K[kv]) / 8.0 - lse64)
        keep = torch.from_numpy(od.keep(p, KEY, (rows * s + kv).astype(np.uint64))).double()
        pk = prob * keep * scale
        assert l2(d_qkv[kv, 2 * d:], pk @ dO) < 3e-2, kv
        ds = prob * ((dO @ V[kv]) * keep * scale - dlt_all)
        assert l2(d_qkv[kv, d:2 * d], (ds @ Q) / 8.0) < 3e-2, kv
