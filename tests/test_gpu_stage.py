"""Stage-level parity on the GPU: the engine (HIP kernels through the C ABI) against the CPU
oracle stage on the same seeded inputs -- loss, parameter gradients, input gradients, the
bit-exactness of redundant forwards, failover promotion and the optimizer step.

Tolerances (of the tensor's own scale): fp32 1e-5 on activations / 1e-4 on accumulated
gradients (different summation order over 2048 rows x 8 micro-batches), bf16 2e-2."""
import numpy as np
import pytest
import torch

import bamboo_amd
from bamboo_amd import LayerSpec, PipelineModule, SeededActivationQueue, TransformerLayer
from oracle import layers as ol
from oracle.stage import OraclePeer, OracleStage

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def rel_err(got, ref, floor=1e-30):
    """fp32 results: max-abs error over the tensor's max; bf16 results (every intermediate is
    rounded to 8 bits of mantissa between kernels): relative L2 error, the 2e-2 of the spec."""
    lowp = got.dtype == torch.bfloat16 or getattr(rel_err, "lowp", False)
    got, ref = got.double().cpu(), ref.double().cpu()
    if lowp:
        return float((got - ref).norm() / ref.norm().clamp_min(floor * ref.numel() ** 0.5))
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(floor))


def grad_floor(ref_grads):
    """Some gradients are zero by construction (the key bias: softmax is invariant to a constant
    added to every key score), so errors are measured against at least 1e-3 of the largest
    gradient of the stage."""
    return 1e-3 * max(float(g.abs().max()) for g in ref_grads.values())


def build(hidden, heads, ffn, layers_per_stage, stages, stage_id, mb, M, seq, dtype, variant, rl, eager,
          grad_mode="queue", rc_stream=False, key_len_range=None, checkpoint_interval=0, loss_fn=None, **engine_kwargs):
    specs = [LayerSpec(TransformerLayer, hidden, heads, ffn, **variant) for _ in range(layers_per_stage * stages)]
    model = PipelineModule(specs, num_stages=stages, partition_method="uniform", stage_id=stage_id, dtype=dtype, device=DEV,
                           activation_checkpoint_interval=checkpoint_interval, loss_fn=loss_fn)
    q = SeededActivationQueue((mb, seq, hidden), dtype, M, stage_ids=[stage_id, (stage_id + 1) % stages], seed=7,
                              grad_mode=grad_mode, device=DEV, key_len_range=key_len_range)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M,
           "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine_kwargs.setdefault("install_signal_handler", False)
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=rl, eager_recovery=eager,
                                            activation_queue=q, rc_stream=rc_stream, **engine_kwargs)
    return engine, q


def oracle_for(engine, q, variant, hidden, heads, ffn, layers_per_stage, stages, stage_id, M, rl, eager, dtype=torch.float64):
    cfg = ol.TransformerCfg(hidden=hidden, heads=heads, ffn=ffn, **variant)
    parts = [i * layers_per_stage for i in range(stages + 1)]
    st = OracleStage(cfg, parts, stage_id, M, dtype=dtype, redundancy_level=rl, eager=eager)
    # the oracle starts from exactly the engine's (possibly bf16-rounded) compute weights
    for sid in list(st.params):
        sp = engine.module.stage_params[sid]
        named = sp.named(sp.compute)
        for key, t in st.named_params(sid).items():
            with torch.no_grad():
                t.copy_(named[key].to(dtype).cpu())
    acts = [a.to(dtype).cpu() for a in q.activations]
    kl = None if q.key_lens is None else [k.cpu() for k in q.key_lens]
    if q.grad_mode == "queue":
        peer = OraclePeer(acts, M, grads={s: [g.to(dtype).cpu() for g in gs] for s, gs in q.grads.items()}, key_lens=kl)
    else:
        peer = OraclePeer(acts, M, targets={s: [t.to(dtype).cpu() for t in ts] for s, ts in q.targets.items()}, key_lens=kl)
    return st, peer


def relu_decisions(engine, stage_ids, M, mb):
    """{(stage, k): per-layer ReLU decisions} read back from the engine's stash after a batch: what each ReLU of
    the low-precision run decided on its own rounded pre-activation (``oracle.layers.activation``)."""
    out = {}
    for s_ in stage_ids:
        for k in range(M):
            per_layer = []
            for st in engine.module._stash[s_][k]:
                if "act" in st:                         # transformer layer: relu(u) of the feed-forward
                    per_layer.append((st["act"] > 0).view(mb, -1, st["act"].shape[1]).cpu())
                else:                                   # bottleneck: three ReLUs, NHWC rows -> NCHW
                    nchw = lambda t: (t > 0).view(mb, int(round((t.shape[0] // mb) ** 0.5)), -1, t.shape[1]).permute(0, 3, 1, 2).cpu()
                    per_layer.append((nchw(st["a1"]), nchw(st["a2"]), nchw(st["out"])))
            out[(s_, k)] = per_layer
    return out


class ReluHandover:
    """Guard of the hand-over of the GPU's ReLU decisions to the oracle (bf16 ReLU layers and bottleneck blocks).

    The masked oracle run measures the kernels' arithmetic at the 2e-2 bar, but would also follow a kernel that
    zeroed (or passed) activations it should not.  So every ReLU evaluated with handed-in decisions is audited
    (``oracle.layers.RELU_AUDIT``): the decisions may differ from the oracle's own ``u > 0`` on under 1 % of the
    elements, and only where the oracle's |u| is below 2e-2 of the tensor's largest |u|: a decision can flip only
    where the low-precision pre-activation is off by more than |u|, and 2e-2 of the tensor's scale is the largest
    element-wise error the bf16 bar grants any tensor (bf16 storage of the operands upstream: 8 bits of mantissa,
    2^-9 relative per stored value, a few stored values deep, amplified by 1/sigma in a BatchNorm).  For scale: a
    ReLU that decided at random would differ on half of the elements, one that was off by a tenth of the tensor's
    spread on a few per cent, with |u| up to that tenth.  And a second oracle run that makes its OWN decisions must
    still agree with the GPU at the looser bars ``LOOSE_ACT`` / ``LOOSE_GRAD`` (a flipped decision moves an
    activation by less than its rounding error, but switches that element's gradient on or off)."""

    def __init__(self, st, peer):
        import copy
        self.own_st, self.own_peer = copy.deepcopy(st), copy.deepcopy(peer)      # before any run: clean gradients
        ol.RELU_AUDIT = self.audit = []

    def check(self, max_fraction=0.01, max_rel=2e-2):
        ol.RELU_AUDIT = None
        assert self.audit, "no ReLU was evaluated with handed-in decisions"
        total, differ = sum(a[0] for a in self.audit), sum(a[1] for a in self.audit)
        assert differ < max_fraction * total, (differ, total)
        for numel, n_diff, worst, top in self.audit:
            assert n_diff < max_fraction * numel, (n_diff, numel)
            assert worst <= max_rel * top, (worst, top, n_diff, numel)
        print(f"relu hand-over: {differ} of {total} decisions differ ({100.0 * differ / total:.3f} %), largest |u| among "
              f"them {max(a[2] / a[3] for a in self.audit):.5f} of its tensor's largest")
        return differ / total

    def own_run(self):
        """The oracle with its own decisions: (buffers, info, stage)."""
        assert not self.own_peer.relu_masks
        bufs, info = self.own_st.run_batch(self.own_peer, optimizer_step=False)
        return bufs, info, self.own_st


def max_err(got, ref):
    """Largest element-wise error over the reference's largest magnitude."""
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / ref.abs().max().clamp_min(1e-30))


def snapshot_grads(engine, sid):
    return {k: v.clone() for k, v in engine.module.get_named_grad(sid)}


class NoStep:
    """Keeps the optimizer from consuming the gradients so they can be inspected."""

    def __init__(self, engine):
        self.engine = engine

    def __enter__(self):
        self.saved = self.engine._exec_optimizer_step
        self.engine._INSTRUCTION_MAP = dict(self.engine._INSTRUCTION_MAP)
        from bamboo_amd import schedule
        self.engine._INSTRUCTION_MAP[schedule.OptimizerStep] = lambda self_: None
        return self

    def __exit__(self, *a):
        del self.engine._INSTRUCTION_MAP


REFERENCE_VARIANT = dict(activation="relu", ln="annotated", mask="none")
# bars of the comparison with an oracle that makes its own ReLU decisions (see ReluHandover): activations stay at the
# bf16 bar; gradients get room for the elements whose decision differs -- 0.1-0.26 % of the decisions per ReLU, each
# switching a whole gradient element on or off, six ReLUs deep in a two-block stage and spread over the batch by the
# BatchNorm backward: relative L2 up to sqrt(6 x 0.0025) = 0.12 (measured 0.10-0.11 on the bottleneck stages, 0.03
# on the transformer's single ReLU per layer)
LOOSE_ACT, LOOSE_GRAD = 2e-2, 2e-1
GPT_VARIANT = dict(activation="gelu_tanh", ln="standard", mask="causal")
BERT_VARIANT = dict(activation="gelu_tanh", ln="standard", mask="key_padding")


@pytest.mark.parametrize("variant,klr", [(REFERENCE_VARIANT, None), (GPT_VARIANT, None), (BERT_VARIANT, (5, 64))],
                         ids=["reference", "gpt", "bert"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_stage_matches_oracle_with_rc(hiplib, variant, klr, dtype):
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, variant, 1, True, key_len_range=klr)
    st, peer = oracle_for(engine, q, variant, hid, heads, ffn, L, S, sid, M, 1, True)
    with NoStep(engine):
        engine._reserve_pipe_buffers(M)
        keep = {}
        orig_clean = engine._clean_pipe_buffers
        engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
        engine.train_batch()
        engine._clean_pipe_buffers = orig_clean
    torch.cuda.synchronize()
    if dtype == torch.bfloat16 and variant["activation"] == "relu":
        # ReLU'(u) is discontinuous: the ~0.2 % of pre-activations closer to zero than their bf16 rounding
        # error would take the other branch in an fp64 run.  The oracle is handed the decisions the GPU made,
        # so that the 2e-2 below measures the kernels' arithmetic
        handover = ReluHandover(st, peer)
        peer.relu_masks = relu_decisions(engine, [sid, sid + 1], M, mb)
    else:
        handover = None
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    t_act = 1e-5 if dtype == torch.float32 else 2e-2
    t_grad = 1e-4 if dtype == torch.float32 else 2e-2
    rel_err.lowp = dtype == torch.bfloat16          # fp32 gradient arenas of a bf16 run
    for k in range(M):
        assert rel_err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().view(mb * seq, hid)) < t_act
        assert rel_err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().view(mb * seq, hid)) < t_act
        assert rel_err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].view(mb * seq, hid)) < t_grad
        if dtype == torch.bfloat16:     # beside the L2 bars: no single element off by more than 5e-2 of the tensor's scale
            assert max_err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().view(mb * seq, hid)) < 5e-2
            assert max_err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().view(mb * seq, hid)) < 5e-2
    ref_grads = st.named_grads(sid)
    for name, g in engine.module.get_named_grad(sid):
        assert rel_err(g, ref_grads[name], grad_floor(ref_grads)) < t_grad, name
    if handover is not None:
        handover.check()
        own_bufs, _, own_st = handover.own_run()
        for k in range(M):
            assert rel_err(keep[f"output_{sid}"][k], own_bufs["out"][(sid, k)].detach().view(mb * seq, hid)) < LOOSE_ACT
            assert rel_err(keep[f"input_grad_{sid}"][k], own_bufs["sent_grad"][(sid, k)].view(mb * seq, hid)) < LOOSE_GRAD
        own_grads = own_st.named_grads(sid)
        for name, g in engine.module.get_named_grad(sid):
            assert rel_err(g, own_grads[name], grad_floor(own_grads)) < LOOSE_GRAD, name
    # shadow parameters receive no gradient from redundant forwards
    for name, g in engine.module.get_named_grad(sid + 1):
        assert float(g.abs().max()) == 0.0


@pytest.mark.parametrize("rc_stream", [False, True], ids=["one-stream", "rc-stream"])
def test_rc_forward_bit_exact_and_rc_neutral(hiplib, rc_stream):
    """(1) The redundant forward of the shadow layers is bit-identical to a normal forward of the
    same layers on the same input; (2) switching RC on changes nothing in the own results."""
    hid, heads, ffn, L, S, sid, mb, M, seq = 256, 4, 512, 2, 4, 1, 2, 6, 128
    dtype = torch.bfloat16
    outs = {}
    for tag, (rl, eager) in {"off": (0, False), "on": (1, True)}.items():
        engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, rl, eager, rc_stream=rc_stream)
        with NoStep(engine):
            keep = {}
            engine._clean_pipe_buffers = lambda: keep.update({k: [None if t is None else t.clone() for t in v]
                                                              for k, v in engine.pipe_buffers.items()})
            engine.train_batch()
        torch.cuda.synchronize()
        outs[tag] = (keep, snapshot_grads(engine, sid), engine)
    for k in range(M):
        assert torch.equal(outs["off"][0][f"output_{sid}"][k], outs["on"][0][f"output_{sid}"][k])
        assert torch.equal(outs["off"][0][f"input_grad_{sid}"][k], outs["on"][0][f"input_grad_{sid}"][k])
    for name in outs["off"][1]:
        assert torch.equal(outs["off"][1][name], outs["on"][1][name]), name
    # normal forward of the shadow stage's layers, as a stage of its own, on the own outputs
    keep, _, engine = outs["on"]
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
    model2 = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid + 1, dtype=dtype, device=DEV)
    ctx2 = model2.prepare_context([sid + 1], mb, seq)
    model2.allocate_stash(sid + 1, ctx2, 1)
    for k in range(M):
        normal = model2.forward(keep[f"output_{sid}"][k], sid + 1, slot=0, ctx=ctx2)
        torch.cuda.synchronize()
        assert torch.equal(normal, keep[f"output_{sid + 1}"][k]), f"micro-batch {k}"


@pytest.mark.parametrize("dead_from,dropout", [(0, 0.0), (2, 0.0), (3, 0.0), (2, 0.1)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_failover_promotion_matches_oracle(hiplib, dead_from, dtype, dropout):
    """The successor is preempted at micro-batch ``dead_from``: the engine promotes the shadow
    layers, replays the successor's backward passes from the stashed redundant activations and
    ends the batch with the gradients of both stages (oracle: same stream on CPU autograd).  With dropout the
    promoted layers' backward passes make the decisions of the redundant forwards again."""
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64
    variant = dict(GPT_VARIANT, dropout=dropout)
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, variant, 1, True, grad_mode="mse")
    st, peer = oracle_for(engine, q, variant, hid, heads, ffn, L, S, sid, M, 1, True)
    # while alive, the successor returns the true gradients of the downstream loss
    true_grads = []
    for k in range(M):
        o1 = st.forward(peer.activations[k], sid, drop_id=(0, k)).detach().requires_grad_(True)
        o2 = st.forward(o1, sid + 1, drop_id=(0, k))
        (torch.nn.functional.mse_loss(o2, peer.targets[sid + 1][k]) / M).backward()
        true_grads.append(o1.grad)
    for s_ in st.params.values():
        for p in s_:
            for t in p.values():
                t.grad = None
    peer.targets = {sid + 1: peer.targets[sid + 1]}
    peer.grads = {sid: true_grads}
    peer.dead_from, peer.dead_stage = dead_from, sid
    st.run_batch(peer, optimizer_step=False)

    q.grad_mode = "mse"
    q.set_grads(sid, [g.view(mb, seq, hid) for g in true_grads])
    q.targets.pop(sid)                      # own outputs go to a live successor, not to a loss head
    orig_send = q.send_activation

    def send(k, tensor, stage_id, stream=None):
        if stage_id == sid:
            q._check_alive(k, stage_id)
            return
        return orig_send(k, tensor, stage_id, stream=stream)
    q.send_activation = send
    q.preempt_successor(dead_from, sid)
    with NoStep(engine):
        loss = engine.train_batch()
    assert engine.stage_ids == [sid, sid + 1] and engine.r_stage_ids == []
    tg = 1e-4 if dtype == torch.float32 else 2e-2
    rel_err.lowp = dtype == torch.bfloat16
    for s_ in (sid, sid + 1):
        ref = st.named_grads(s_)
        for name, g in engine.module.get_named_grad(s_):
            assert rel_err(g, ref[name], grad_floor(ref)) < tg, (s_, name)
    assert abs(float(loss) - float(peer.loss) / M) < tg * max(1.0, float(peer.loss) / M)
    # next batch runs as a merged two-stage process from step 0
    q.revive()
    engine.train_batch()
    assert engine.global_steps == 1 or engine.global_steps == 2


@pytest.mark.parametrize("dead_from", [0, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_failover_onto_the_last_stage_computes_the_loss(hiplib, dead_from, dtype):
    """The stage in front of the LAST stage absorbs it: micro-batches whose last-stage forward ran as a
    redundant forward still get their loss and its gradient in the replay (the reference recomputes that
    forward, engine.py:1646-1663), so every BackwardPass of the absorbed stage finds a gradient and the
    reported loss covers all micro-batches."""
    from bamboo_amd import MSELoss
    hid, heads, ffn, L, S, mb, M, seq = 128, 2, 256, 2, 4, 2, 4, 64
    sid = S - 2
    g = torch.Generator().manual_seed(21)
    labels = [torch.randn(mb, seq, hid, generator=g) for _ in range(M)]
    data = [(torch.zeros(1), y.to(dtype)) for y in labels]
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, True, loss_fn=MSELoss(),
                      training_data=data * 4)
    st, peer = oracle_for(engine, q, GPT_VARIANT, hid, heads, ffn, L, S, sid, M, 1, True)
    olabels = [y.to(dtype).double() for y in labels]
    true_grads = []
    for k in range(M):
        o1 = st.forward(peer.activations[k], sid).detach().requires_grad_(True)
        (torch.nn.functional.mse_loss(st.forward(o1, sid + 1), olabels[k]) / M).backward()
        true_grads.append(o1.grad)
    for s_ in st.params.values():
        for p in s_:
            for t in p.values():
                t.grad = None
    peer.grads, peer.labels = {sid: true_grads}, olabels
    peer.dead_from, peer.dead_stage = dead_from, sid
    st.run_batch(peer, optimizer_step=False)

    q.set_grads(sid, [g_.view(mb, seq, hid) for g_ in true_grads])
    q.preempt_successor(dead_from, sid)
    with NoStep(engine):
        loss = engine.train_batch()
    torch.cuda.synchronize()
    assert engine.stage_ids == [sid, sid + 1] and engine.is_last_stage() is False
    tg = 1e-4 if dtype == torch.float32 else 2e-2
    rel_err.lowp = dtype == torch.bfloat16
    for s_ in (sid, sid + 1):
        ref = st.named_grads(s_)
        for name, g_ in engine.module.get_named_grad(s_):
            assert rel_err(g_, ref[name], grad_floor(ref)) < tg, (s_, name)
    assert float(peer.loss) > 0 and abs(float(loss) - float(peer.loss) / M) < tg * float(peer.loss) / M
    # the next batch runs both stages from step 0, loss head included
    q.revive()
    loss2 = engine.train_batch()
    assert abs(float(loss2) - float(loss)) < 0.1 * float(loss)


@pytest.mark.parametrize("dtype,cin,cmid", [(torch.float32, 64, 16), (torch.bfloat16, 64, 16), (torch.bfloat16, 512, 128),
                                            (torch.bfloat16, 1024, 256)],
                         ids=["fp32", "bf16", "bf16-implicit-gemm", "bf16-resnet152-conv4-shape"])
def test_resnet_stage_matches_oracle_with_rc(hiplib, dtype, cin, cmid):
    """Bottleneck stage (conv 1x1 -> 3x3 -> 1x1, train-mode BatchNorm, ReLU, identity shortcut) with
    redundant forwards of the shadow blocks, against the torch conv2d / batch_norm oracle.  With 128 middle
    channels the 3x3 convolution and its input gradient run as implicit GEMMs, with 16 through the patch matrix.
    The last case is the benchmark's own block shape: 32 images of 14x14, 1024 -> 256 -> 256 -> 1024 channels
    (one own and one shadow block, two micro-batches: the CPU oracle runs it in fp64)."""
    from bamboo_amd import BottleNeck
    side, L, S, sid, mb, M = 6, 2, 4, 1, (8 if cmid == 128 else 4), 4     # 288 pixels: whole 32-pixel k-tiles for the weight gradient
    if cin == 1024:
        side, L, mb, M = 14, 1, 32, 2
    assert hiplib.conv3x3_supported(dtype, hiplib.CONV_DGRAD, mb, side, side, cmid, cmid) == (cmid >= 128)
    specs = [LayerSpec(BottleNeck, cin, cmid, height=side, width=side) for _ in range(L * S)]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
    q = SeededActivationQueue((mb, side * side, cin), dtype, M, stage_ids=[sid, sid + 1], seed=9, device=DEV)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                            activation_queue=q, install_signal_handler=False)
    ocfg = ol.BottleneckCfg(in_channels=cin, mid_channels=cmid)
    st = OracleStage(ocfg, [i * L for i in range(S + 1)], sid, M, dtype=torch.float64, redundancy_level=1, eager=True)
    for s_ in list(st.params):
        sp = engine.module.stage_params[s_]
        named = sp.named(sp.compute)
        for key, t in st.named_params(s_).items():
            src = named[key].double().cpu()
            if t.dim() == 4:      # arena keeps [O, kh, kw, I]; the oracle the reference's [O, I, kh, kw]
                src = src.view(t.shape[0], t.shape[2], t.shape[3], t.shape[1]).permute(0, 3, 1, 2)
            with torch.no_grad():
                t.copy_(src.reshape(t.shape))
    peer = OraclePeer([a.double().cpu() for a in q.activations], M,
                      grads={s_: [g.double().cpu() for g in gs] for s_, gs in q.grads.items()})
    rel_err.lowp = dtype == torch.bfloat16
    keep = {}
    with NoStep(engine):
        engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
        engine.train_batch()
    torch.cuda.synchronize()
    if dtype == torch.bfloat16:
        # every block has three ReLUs; the oracle takes the decisions the GPU made at each of them (see the
        # transformer ReLU case), so the bf16 bar stays at 2e-2
        handover = ReluHandover(st, peer)
        peer.relu_masks = relu_decisions(engine, [sid, sid + 1], M, mb)
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    t_act = 1e-5 if dtype == torch.float32 else 2e-2
    t_grad = 1e-4 if dtype == torch.float32 else 2e-2
    rows = mb * side * side

    def compare(bufs, stage, t_act, t_grad, elementwise):
        for k in range(M):
            assert rel_err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().reshape(rows, cin)) < t_act
            assert rel_err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().reshape(rows, cin)) < t_act
            assert rel_err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].reshape(rows, cin)) < t_grad
            if elementwise:
                assert max_err(keep[f"output_{sid}"][k], bufs["out"][(sid, k)].detach().reshape(rows, cin)) < 5e-2
                assert max_err(keep[f"output_{sid + 1}"][k], bufs["out"][(sid + 1, k)].detach().reshape(rows, cin)) < 5e-2
        ref = stage.named_grads(sid)
        for name, g in engine.module.get_named_grad(sid):
            r = ref[name]
            if r.dim() == 4:
                r = r.permute(0, 2, 3, 1)
            assert rel_err(g, r.reshape(g.shape), grad_floor(ref)) < t_grad, name
    compare(bufs, st, t_act, t_grad, dtype == torch.bfloat16)
    if dtype == torch.bfloat16:
        handover.check()
        own_bufs, _, own_st = handover.own_run()
        compare(own_bufs, own_st, LOOSE_ACT, LOOSE_GRAD, False)
    # where the kernels exist (bf16, whole 64-channel k-tiles) the BatchNorm backward sums came out of the epilogues of
    # the kernels that write the gradients, also across the boundary between the stage's two blocks; elsewhere from
    # the reduction pass
    fused = {k[0]: v for layer in engine.module.func_buckets[sid] for k, v in layer._stats_ok.items() if k[0] in ("bn_bwd", "sink")}
    if cmid == 128:
        assert fused == {"bn_bwd": True, "sink": True}
    elif cmid == 16:
        assert not any(fused.values())
    # redundant forwards left the shadow blocks' running statistics alone; own blocks updated theirs M times
    for layer in engine.module.func_buckets[sid + 1]:
        assert layer.running is None
    for layer in engine.module.func_buckets[sid]:
        assert float(layer.running[1][0].abs().max()) > 0


DOWNSAMPLING_NET = [  # (in, mid, stride) of every block: widening, down-sampling and identity-shortcut blocks mixed
    (32, 16, 1), (64, 16, 1),            # stage 0: projection 32 -> 64, identity
    (64, 32, 2), (128, 32, 1),           # stage 1: 16x16 -> 8x8 with 64 -> 128 channels, identity
    (128, 64, 1), (256, 64, 2),          # stage 2: widening projection at stride 1, then 8x8 -> 4x4
    (256, 64, 1), (256, 64, 1)]          # stage 3
# one block per stage: what bf16 storage between the kernels leaves of a gradient that has crossed two blocks
# forward and two backward stays inside the 2e-2 bar (across four blocks it reaches 1.8 % on the activations alone)
SHALLOW_DOWNSAMPLING_NET = [(32, 16, 1), (64, 32, 2), (128, 64, 2), (256, 64, 1)]


@pytest.mark.parametrize("dtype,net,dead_from", [(torch.float32, DOWNSAMPLING_NET, None), (torch.float32, DOWNSAMPLING_NET, 1),
                                                 (torch.bfloat16, DOWNSAMPLING_NET, None),
                                                 (torch.bfloat16, SHALLOW_DOWNSAMPLING_NET, 1)],
                         ids=["fp32-rc", "fp32-failover", "bf16-rc", "bf16-failover"])
def test_resnet_stage_with_projection_shortcuts_matches_oracle(hiplib, dtype, net, dead_from):
    """Bottleneck blocks with the projection shortcut (conv1x1(stride) + BatchNorm, resnet.py:68-72) and a stride on
    the 3x3 convolution: the own stage halves the image and doubles the channels, the shadowed stage widens at
    stride 1 and / or halves again, so rows and features differ at every stage boundary (and, in the two-block
    stages, inside a stage).  Outputs, input gradients and all parameter gradients against the conv2d / batch_norm
    oracle, with redundant forwards, and through a failover that promotes the shadowed stage."""
    from bamboo_amd import BottleNeck
    S, sid, mb, M, side = 4, 1, 8, 4, 16     # the smallest BatchNorm still sees 128 pixels
    L = len(net) // S
    specs = [LayerSpec(BottleNeck, ci, cm, stride=st_, height=None, width=None) for ci, cm, st_ in net]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
    seq_of = lambda n_blocks: side * side // 4 ** sum(st_ == 2 for _, _, st_ in net[:n_blocks])
    shapes = {s_: (mb, seq_of((s_ + 1) * L), 4 * net[(s_ + 1) * L - 1][1]) for s_ in (sid, sid + 1)}
    q = SeededActivationQueue((mb, side * side, 64), dtype, M, stage_ids=[sid, sid + 1], seed=19, device=DEV, out_shapes=shapes)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                            activation_queue=q, install_signal_handler=False)
    assert model.func_buckets[sid][0].projection and model.func_buckets[sid][0].stride == 2
    if L == 2:
        assert model.stage_seq[sid] == [256, 64, 64] and model.stage_seq[sid + 1] == [64, 64, 16]
        assert shapes == {sid: (mb, 64, 128), sid + 1: (mb, 16, 256)}
    ocfgs = [ol.BottleneckCfg(in_channels=ci, mid_channels=cm, stride=st_) for ci, cm, st_ in net]
    st = OracleStage(ocfgs, [i * L for i in range(S + 1)], sid, M, dtype=torch.float64, redundancy_level=1, eager=True)
    for s_ in list(st.params):
        sp = engine.module.stage_params[s_]
        named = sp.named(sp.compute)
        assert set(named) == set(st.named_params(s_))
        for key, t in st.named_params(s_).items():
            src = named[key].double().cpu()
            if t.dim() == 4:      # arena keeps [O, kh, kw, I]; the oracle the reference's [O, I, kh, kw]
                src = src.view(t.shape[0], t.shape[2], t.shape[3], t.shape[1]).permute(0, 3, 1, 2)
            with torch.no_grad():
                t.copy_(src.reshape(t.shape))
    peer = OraclePeer([a.double().cpu() for a in q.activations], M,
                      grads={s_: [g.double().cpu() for g in gs] for s_, gs in q.grads.items()})
    if dead_from is not None:
        peer.dead_from, peer.dead_stage = dead_from, sid
        q.preempt_successor(dead_from, sid)
    rel_err.lowp = dtype == torch.bfloat16
    keep = {}
    with NoStep(engine):
        clean = engine._clean_pipe_buffers
        engine._clean_pipe_buffers = lambda: (keep.update({k: list(v) for k, v in engine.pipe_buffers.items()}), clean())
        engine.train_batch()
    torch.cuda.synchronize()
    if dtype == torch.bfloat16:
        handover = ReluHandover(st, peer)
        peer.relu_masks = relu_decisions(engine, [sid, sid + 1], M, mb)
    bufs, info = st.run_batch(peer, optimizer_step=False)
    assert (info["failed_step"] is not None) == (dead_from is not None)
    assert engine.stage_ids == ([sid, sid + 1] if dead_from is not None else [sid])
    t_act = 1e-5 if dtype == torch.float32 else 2e-2
    t_grad = 1e-4 if dtype == torch.float32 else 2e-2

    def compare(bufs, stage, t_act, t_grad, elementwise):
        for k in range(M):
            for s_ in (sid, sid + 1):
                want = bufs["out"][(s_, k)].detach()
                assert rel_err(keep[f"output_{s_}"][k], want.reshape(-1, want.shape[-1])) < t_act, (s_, k)
                if elementwise:
                    assert max_err(keep[f"output_{s_}"][k], want.reshape(-1, want.shape[-1])) < 5e-2, (s_, k)
            want = bufs["sent_grad"][(sid, k)]
            assert rel_err(keep[f"input_grad_{sid}"][k], want.reshape(-1, want.shape[-1])) < t_grad, k
        for s_ in engine.stage_ids:
            ref = stage.named_grads(s_)
            for name, g in engine.module.get_named_grad(s_):
                r = ref[name]
                if r.dim() == 4:
                    r = r.permute(0, 2, 3, 1)
                assert rel_err(g, r.reshape(g.shape), grad_floor(ref)) < t_grad, (s_, name)
    compare(bufs, st, t_act, t_grad, dtype == torch.bfloat16)
    if dtype == torch.bfloat16:
        handover.check()
        own_bufs, own_info, own_st = handover.own_run()
        assert (own_info["failed_step"] is not None) == (dead_from is not None)
        compare(own_bufs, own_st, LOOSE_ACT, LOOSE_GRAD, False)
    # the shortcut's BatchNorm keeps running statistics like the others
    own = engine.module.func_buckets[sid][0]
    assert float(own.running["shortcut"][0].abs().max()) > 0


@pytest.mark.parametrize("dead_from", [0, 2])
def test_lazy_recovery_failover(hiplib, dead_from):
    """redundancy_level=1 without eager recovery: no redundant forwards (only pings); the shadow stage exists
    as CPU parameter mirrors and is materialised at the failover, its forwards are recomputed in the replay."""
    rel_err.lowp = False
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64
    dtype = torch.float32
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, False, grad_mode="mse")
    assert engine.r_stage_ids == [sid + 1] and (sid + 1) not in engine.module.func_buckets
    assert all(t.device.type == "cpu" and float(t.abs().max()) == 0 for t in engine.param_buffers[sid + 1].values())
    # what a weight synchronisation would have put into the mirrors: the successor's parameters
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
    succ = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid + 1, dtype=dtype, device=DEV)
    for name, p in succ.get_named_param(sid + 1):
        engine.param_buffers[sid + 1][name].copy_(p.cpu())
    st, peer = oracle_for(engine, q, GPT_VARIANT, hid, heads, ffn, L, S, sid, M, 1, False)
    true_grads = []
    st.build(sid + 1)
    for k in range(M):
        o1 = st.forward(peer.activations[k], sid).detach().requires_grad_(True)
        (torch.nn.functional.mse_loss(st.forward(o1, sid + 1), peer.targets[sid + 1][k]) / M).backward()
        true_grads.append(o1.grad)
    for s_ in st.params.values():
        for p in s_:
            for t in p.values():
                t.grad = None
    peer.targets = {sid + 1: peer.targets[sid + 1]}
    peer.grads = {sid: true_grads}
    peer.dead_from, peer.dead_stage = dead_from, sid
    st.run_batch(peer, optimizer_step=False)

    q.set_grads(sid, [g.view(mb, seq, hid) for g in true_grads])
    q.targets.pop(sid)
    orig_send = q.send_activation
    q.send_activation = lambda k, t, stage_id, stream=None: (q._check_alive(k, stage_id) if stage_id == sid
                                                              else orig_send(k, t, stage_id, stream=stream))
    q.preempt_successor(dead_from, sid)
    with NoStep(engine):
        loss = engine.train_batch()
    assert engine.stage_ids == [sid, sid + 1]
    for s_ in (sid, sid + 1):
        ref = st.named_grads(s_)
        for name, g in engine.module.get_named_grad(s_):
            assert rel_err(g, ref[name], grad_floor(ref)) < 1e-4, (s_, name)
    assert abs(float(loss) - float(peer.loss) / M) < 1e-4 * max(1.0, float(peer.loss) / M)


@pytest.mark.parametrize("ckpt", [0, 1], ids=["full-stash", "checkpointed"])
@pytest.mark.parametrize("rc_stream", [False, True], ids=["one-stream", "rc-stream"])
@pytest.mark.parametrize("variant,klr", [(GPT_VARIANT, None), (BERT_VARIANT, (5, 64))], ids=["gpt", "bert"])
def test_graph_replay_equals_eager(hiplib, variant, klr, rc_stream, ckpt):
    """Forward / backward launch sequences replayed as HIP graphs: five batches with optimizer steps
    (eager work and synchronisation between the replays), loss after every batch and the weights at
    the end bit-equal to an engine that launches every kernel itself.  Batch 1 runs eagerly, batch 2
    captures, batches 3-5 replay."""
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64
    dtype = torch.bfloat16
    eager_engine, _ = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, variant, 1, True, grad_mode="mse",
                            rc_stream=rc_stream, key_len_range=klr, checkpoint_interval=ckpt)
    ref_losses = []
    for _ in range(5):
        ref_losses.append(float(eager_engine.train_batch()))
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        with pytest.raises(bamboo_amd.PipelineError):
            pass_default = torch.cuda.default_stream()
            with torch.cuda.stream(pass_default):
                build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, variant, 1, True, grad_mode="mse", use_graphs=True)
        engine, _ = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, variant, 1, True, grad_mode="mse",
                          rc_stream=rc_stream, key_len_range=klr, use_graphs=True, checkpoint_interval=ckpt)
        torch.cuda.synchronize()
        losses = []
        for _ in range(5):
            losses.append(float(engine.train_batch()))
            torch.cuda.synchronize()
    assert losses == ref_losses
    assert len(engine._graphs) == 3 * M and all(isinstance(v, tuple) for v in engine._graphs.values())
    for s_ in (sid, sid + 1):
        a, b = engine.module.stage_params[s_], eager_engine.module.stage_params[s_]
        assert torch.equal(a.master, b.master) and torch.equal(a.compute, b.compute)
    assert losses[4] != losses[0]


def test_graph_replay_equals_eager_on_a_resnet_stage(hiplib):
    """The same for a bottleneck stage of the widths whose backward takes the BatchNorm sums from GEMM epilogues and
    hands a gradient from block to block with the next block's mask and sums: four batches with optimizer steps,
    weights, Adam moments and BatchNorm running statistics bit-equal between launching every kernel and replaying
    the captured passes."""
    from bamboo_amd import BottleNeck
    cin, cmid, side, L, S, sid, mb, M = 512, 128, 6, 2, 4, 1, 8, 4
    def make(use_graphs):
        specs = [LayerSpec(BottleNeck, cin, cmid, height=side, width=side) for _ in range(L * S)]
        model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=torch.bfloat16, device=DEV)
        q = SeededActivationQueue((mb, side * side, cin), torch.bfloat16, M, stage_ids=[sid, sid + 1], seed=9, device=DEV)
        cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": True},
               "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}}
        engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                                activation_queue=q, install_signal_handler=False, use_graphs=use_graphs)
        for _ in range(4):
            engine.train_batch()
            torch.cuda.synchronize()
        return engine
    eager = make(False)
    side_stream = torch.cuda.Stream()
    with torch.cuda.stream(side_stream):
        graphed = make(True)
    torch.cuda.synchronize()
    assert graphed._graphs and all(isinstance(v, tuple) for v in graphed._graphs.values())
    assert any(k[0] == "sink" and v for layer in graphed.module.func_buckets[sid] for k, v in layer._stats_ok.items())
    a, b = graphed.module.stage_params[sid], eager.module.stage_params[sid]
    assert torch.equal(a.master, b.master) and torch.equal(a.exp_avg_sq, b.exp_avg_sq)
    for la, lb in zip(graphed.module.func_buckets[sid], eager.module.func_buckets[sid]):
        ra, rb = la._running(DEV), lb._running(DEV)
        for idx in ra:
            assert torch.equal(ra[idx][0], rb[idx][0]) and torch.equal(ra[idx][1], rb[idx][1])


@pytest.mark.parametrize("interval", [1, 2, 3])
@pytest.mark.parametrize("rc_stream", [False, True], ids=["one-stream", "rc-stream"])
def test_activation_checkpointing_equals_full_stash(hiplib, interval, rc_stream):
    """activation_checkpoint_interval > 0 (reference module.py:551-573): only the input of every layer group is
    kept per micro-batch and the group's forward runs again in the backward pass.  Losses of batches with
    optimizer steps, a batch that loses the successor at micro-batch 2 (backward of the promoted layers from
    their kept inputs), the batch after it, and all weights are bit-equal to the full stash, which takes
    several times the memory."""
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 3, 4, 1, 2, 4, 64
    dtype = torch.bfloat16
    runs = []
    for every in (0, interval):
        engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, True, grad_mode="mse",
                          rc_stream=rc_stream, checkpoint_interval=every)
        losses = [float(engine.train_batch()) for _ in range(3)]
        q.preempt_successor(2, sid)
        losses += [float(engine.train_batch()), float(engine.train_batch())]
        torch.cuda.synchronize()
        runs.append((engine, losses))
    (full, lf), (ck, lc) = runs
    assert lf == lc and lf[2] != lf[0]
    assert ck.stash_bytes * 2 < full.stash_bytes
    for s_ in (sid, sid + 1):
        a, b = full.module.stage_params[s_], ck.module.stage_params[s_]
        assert torch.equal(a.master, b.master) and torch.equal(a.compute, b.compute)
        assert torch.equal(a.exp_avg, b.exp_avg) and torch.equal(a.exp_avg_sq, b.exp_avg_sq)


@pytest.mark.parametrize("net", ["identity", "identity-wide", "down-sampling"])
def test_activation_checkpointing_resnet_keeps_running_statistics(hiplib, net):
    """Bottleneck stage with checkpoint groups of one block: gradients, outputs and the BatchNorm running
    statistics (updated once per forward, not again by the recomputation) equal the full stash bit for bit; also
    where the kept group inputs differ in rows and channels (blocks with a stride and a projection shortcut), and
    ("wide") where the full stash takes the last BatchNorm's backward sums of the stage's first block from the
    epilogue of the second block's last GEMM while a group of one block makes them in a pass of its own."""
    from bamboo_amd import BottleNeck
    cin, cmid, side, L, S, sid, mb, M = 64, 16, 6, 2, 4, 1, 4, 4
    if net == "identity-wide":
        cin, cmid, mb = 512, 128, 8
    blocks = [(cin, cmid, 1)] * (L * S) if net != "down-sampling" else DOWNSAMPLING_NET
    if net == "down-sampling":
        side = 16
    out_shapes = {s_: (mb, side * side // 4 ** sum(st_ == 2 for _, _, st_ in blocks[:(s_ + 1) * L]), 4 * blocks[(s_ + 1) * L - 1][1])
                  for s_ in (sid, sid + 1)}
    dtype = torch.bfloat16
    runs = []
    for every in (0, 1):
        specs = [LayerSpec(BottleNeck, ci, cm, stride=st_, height=None, width=None) for ci, cm, st_ in blocks]
        model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV,
                               activation_checkpoint_interval=every)
        q = SeededActivationQueue((mb, side * side, cin), dtype, M, stage_ids=[sid, sid + 1], seed=9, device=DEV,
                                  out_shapes=out_shapes)
        cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": True}}
        engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                                activation_queue=q, install_signal_handler=False)
        for _ in range(2):
            engine.train_batch()
        torch.cuda.synchronize()
        runs.append(engine)
    a, b = runs
    if net == "identity-wide":
        sunk = lambda e: [any(k[0] == "sink" and v for k, v in layer._stats_ok.items()) for layer in e.module.func_buckets[sid]]
        assert sunk(a) == [False, True] and sunk(b) == [False, False]
    for s_ in (sid, sid + 1):
        pa, pb = a.module.stage_params[s_], b.module.stage_params[s_]
        assert torch.equal(pa.master, pb.master) and torch.equal(pa.exp_avg_sq, pb.exp_avg_sq)
    for la, lb in zip(a.module.func_buckets[sid], b.module.func_buckets[sid]):
        ra, rb = la._running(DEV), lb._running(DEV)
        for idx in ra:
            assert torch.equal(ra[idx][0], rb[idx][0]) and torch.equal(ra[idx][1], rb[idx][1])
            assert float(ra[idx][0].abs().sum()) > 0      # the running mean has moved off its zero start


@pytest.mark.parametrize("rc_issue", ["reference", "asap", "bubble"])
def test_paced_pipeline_changes_timing_not_results(hiplib, rc_issue):
    """The stage inside the closed-loop pipeline model (receives wait on the host until a 4-stage 1F1B pipeline
    would deliver; redundant forwards on the second stream, placed as the reference places them or issued as soon
    as their input exists): losses and weights after three batches are bit-equal to the always-ready queue, the
    stage really waited, and no batch beat the pipeline's own length."""
    from bamboo_amd.p2p import PacedActivationQueue
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 6, 64
    dtype = torch.bfloat16
    ref_engine, _ = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, True, grad_mode="mse", rc_stream=True)
    ref_losses = [float(ref_engine.train_batch()) for _ in range(3)]
    t_fwd, t_bwd = 2e-3, 4e-3
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
    q = PacedActivationQueue((mb, seq, hid), dtype, M, stage_ids=[sid, sid + 1], stages=S, stage_id=sid, t_fwd=t_fwd,
                             t_bwd=t_bwd, seed=7, grad_mode="mse", device=DEV)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M,
           "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}, "bf16": {"enabled": True}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                            activation_queue=q, rc_stream=True, rc_issue=rc_issue, install_signal_handler=False)
    losses = []
    for _ in range(3):
        losses.append(float(engine.train_batch()))
        # this stage's own passes are far shorter than its neighbours': the batch is at most one slot shorter than
        # a balanced pipeline's (M + S - 1) slots
        assert q.batch_seconds >= (M + S - 2) * (t_fwd + t_bwd)
        assert q.waited > (S - 1) * t_fwd          # at least the warm-up of the pipeline was spent waiting
    assert q.finish() >= 3 * (M + S - 2) * (t_fwd + t_bwd) and q.batches == 3
    torch.cuda.synchronize()
    assert losses == ref_losses
    for s_ in (sid, sid + 1):
        a, b = engine.module.stage_params[s_], ref_engine.module.stage_params[s_]
        assert torch.equal(a.master, b.master) and torch.equal(a.exp_avg_sq, b.exp_avg_sq)
    with pytest.raises(bamboo_amd.PipelineError):
        build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, True, rc_issue="asap")   # needs the second stream


@pytest.mark.parametrize("dead_from", [1, 4])
@pytest.mark.parametrize("rc_issue", ["asap", "bubble"])
def test_failover_with_redundant_forwards_issued_out_of_order(hiplib, rc_issue, dead_from):
    """The successor is lost while redundant forwards are pending, partly issued or ahead of the schedule (issued as
    soon as their input exists, or held back for the bubbles of the paced pipeline): the promoted stage replays what
    is missing as ordinary forwards.  Losses of the failing batch and the one after it, and every parameter of both
    stages after the two optimizer steps, are bit-equal to the same failure under the reference's placement."""
    from bamboo_amd.p2p import PacedActivationQueue
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 6, 64
    dtype = torch.bfloat16

    def run(issue, paced):
        specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
        model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
        kw = dict(stage_ids=[sid, sid + 1], seed=7, grad_mode="mse", device=DEV)
        q = (PacedActivationQueue((mb, seq, hid), dtype, M, stages=S, stage_id=sid, t_fwd=1e-3, t_bwd=2e-3, **kw) if paced
             else SeededActivationQueue((mb, seq, hid), dtype, M, **kw))
        cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M,
               "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}, "bf16": {"enabled": True}}
        engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                                activation_queue=q, rc_stream=True, rc_issue=issue, install_signal_handler=False)
        losses = [float(engine.train_batch())]
        q.preempt_successor(dead_from, sid)
        losses += [float(engine.train_batch()), float(engine.train_batch())]
        torch.cuda.synchronize()
        assert engine.stage_ids == [sid, sid + 1]
        return engine, losses
    ref, ref_losses = run("reference", False)
    eng, losses = run(rc_issue, True)
    assert losses == ref_losses
    for s_ in (sid, sid + 1):
        a, b = eng.module.stage_params[s_], ref.module.stage_params[s_]
        assert torch.equal(a.master, b.master) and torch.equal(a.exp_avg, b.exp_avg) and torch.equal(a.exp_avg_sq, b.exp_avg_sq)


def test_script_layers_taken_over_run_as_the_last_stage(hiplib):
    """The reference script's own layer list -- EncoderLayer modules, the final LayerNorm, ``lambda x: x.sum(-1)``,
    ``nn.MSELoss()`` against [batch, seq] labels (transformer.py:246-264) -- handed over as it is.  The last stage
    (one encoder layer, norm, sum) runs on the HIP kernels; loss, parameter gradients and the gradient sent
    upstream equal torch autograd on the modules themselves (fp32)."""
    from tests.reference_shapes import RefEncoderLayer, RefLayerNorm
    hid, heads, ffn, mb, M, seq = 128, 2, 256, 2, 4, 64
    torch.manual_seed(11)
    mods = [RefEncoderLayer(hid, heads, ffn, 0.0) for _ in range(2)] + [RefLayerNorm(hid)]
    with torch.no_grad():
        for m in mods:
            for prm in m.parameters():
                prm.add_(0.05 * torch.randn_like(prm))
    layers = mods + [lambda x: x.sum(-1)]
    g = torch.Generator().manual_seed(12)
    labels = [torch.randn(mb, seq, generator=g) for _ in range(M)]
    model = PipelineModule(layers, num_stages=2, partition_method="custom", custom_partitions=[0, 1, 4], stage_id=1,
                           loss_fn=torch.nn.MSELoss(), dtype=torch.float32, device=DEV)
    q = SeededActivationQueue((mb, seq, hid), torch.float32, M, stage_ids=[1], seed=5, device=DEV)
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, activation_queue=q, install_signal_handler=False,
                                            training_data=[(torch.zeros(1), y) for y in labels])
    with NoStep(engine):
        loss = engine.train_batch()
    torch.cuda.synchronize()
    total, xgrads = 0.0, []
    for k in range(M):
        x = q.activations[k].cpu().clone().requires_grad_(True)
        out = layers[3](mods[2](mods[1](x)))
        l = torch.nn.functional.mse_loss(out, labels[k])
        (l / M).backward()
        total += float(l)
        xgrads.append(x.grad)
    rel_err.lowp = False
    assert abs(float(loss) - total / M) < 1e-5 * total / M
    ref = {f"{li}.{n}": p.grad for li in (1, 2) for n, p in mods[li].named_parameters()}
    got = dict(engine.module.get_named_grad(1))
    assert set(got) == set(ref)
    floor = grad_floor(ref)
    for name, gr in got.items():
        assert rel_err(gr, ref[name], floor) < 1e-4, name
    for k in range(M):
        assert rel_err(q.sent_grads[(1, k)], xgrads[k].view(mb * seq, hid)) < 1e-4


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_last_stage_with_the_script_tail_matches_oracle(hiplib, dtype):
    """Last stage = transformer layer, final LayerNorm, sum over the hidden dimension, MSE against [batch, seq]
    labels (native layer specs, GPT variant) against the oracle stage with the same tail."""
    from bamboo_amd import FinalLayerNorm, MSELoss, SumLast
    hid, heads, ffn, mb, M, seq = 128, 2, 256, 2, 4, 64
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(2)]
    specs += [LayerSpec(FinalLayerNorm, hid, ln="standard"), LayerSpec(SumLast, hid)]
    model = PipelineModule(specs, num_stages=2, partition_method="custom", custom_partitions=[0, 1, 4], stage_id=1,
                           loss_fn=MSELoss(), dtype=dtype, device=DEV)
    # a final norm with gain 1 and shift 0 sums to zero: move it off that point
    sp = model.stage_params[1]
    gen = torch.Generator().manual_seed(3)
    sp.load({"2.a_2": 1 + 0.3 * torch.randn(hid, generator=gen), "2.b_2": 0.3 * torch.randn(hid, generator=gen)})
    q = SeededActivationQueue((mb, seq, hid), dtype, M, stage_ids=[1], seed=5, device=DEV)
    labels = [torch.randn(mb, seq, generator=gen).to(dtype) for _ in range(M)]
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, activation_queue=q, install_signal_handler=False,
                                            training_data=[(torch.zeros(1), y) for y in labels])
    st = OracleStage(ol.TransformerCfg(hidden=hid, heads=heads, ffn=ffn, **GPT_VARIANT), [0, 1, 4], 1, M, dtype=torch.float64, tail=True)
    named = sp.named(sp.compute)
    for key, t in st.named_params(1).items():
        with torch.no_grad():
            t.copy_(named[key].double().cpu())
    peer = OraclePeer([a.double().cpu() for a in q.activations], M, labels=[y.double() for y in labels])
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    with NoStep(engine):
        loss = engine.train_batch()
    torch.cuda.synchronize()
    tol = 1e-4 if dtype == torch.float32 else 2e-2
    rel_err.lowp = dtype == torch.bfloat16
    assert abs(float(loss) - float(peer.loss) / M) < tol * float(peer.loss) / M
    ref = st.named_grads(1)
    for name, gr in engine.module.get_named_grad(1):
        assert rel_err(gr, ref[name], grad_floor(ref)) < tol, name
    for k in range(M):
        assert rel_err(q.sent_grads[(1, k)], bufs["sent_grad"][(1, k)].view(mb * seq, hid)) < tol


def test_optimizer_step_matches_oracle(hiplib):
    rel_err.lowp = False
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.float32, GPT_VARIANT, 0, False)
    st, peer = oracle_for(engine, q, GPT_VARIANT, hid, heads, ffn, L, S, sid, M, 0, False, dtype=torch.float32)
    before = {k: v.clone() for k, v in engine.module.get_named_param(sid)}
    for _ in range(2):
        engine.train_batch()
        st.run_batch(peer)
    assert engine.global_steps == 2
    ref = st.named_params(sid)
    for name, p in engine.module.get_named_param(sid):
        # Adam's first steps move every weight by ~lr whatever the gradient scale, so compare the
        # movement: |delta - delta_ref| small against lr
        if name.endswith("linears.1.bias"):
            continue    # key bias: exact gradient is zero, Adam normalises pure rounding noise to +-lr
        d, dr = (p - before[name]).cpu(), (ref[name].detach() - before[name].cpu())
        assert float((d - dr).abs().max()) < 2e-4, name
        assert float(d.abs().max()) > 1e-4
    for name, g in engine.module.get_named_grad(sid):
        assert float(g.abs().max()) == 0.0      # zero_grad fused into the optimizer kernel


def test_engine_surface(hiplib):
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 1, 4, 1, 2, 4, 64
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.float32, GPT_VARIANT, 1, True)
    assert (engine.micro_batches, engine.micro_batch_size, engine.stage_id, engine.num_stages) == (M, mb, sid, S)
    assert engine.stage_ids == [sid] and engine.r_stage_ids == [sid + 1] and engine.r_user_stage_ids == [sid - 1]
    assert not engine.is_first_stage() and not engine.is_last_stage()
    for key in (f"input_{sid}", f"output_{sid}", f"input_{sid + 1}", f"output_{sid + 1}", f"input_grad_{sid}", "data", "label"):
        assert key in engine.pipe_buffers
    with pytest.raises(bamboo_amd.PipelineError):
        engine.forward(None)
    with pytest.raises(bamboo_amd.PipelineError):
        engine.backward(None)
    with pytest.raises(bamboo_amd.PipelineError):
        engine.step()
    names = [n for n, _ in engine.module.get_named_param(sid)]
    assert names[0] == "1.sublayer.0.norm.a_2" and "1.self_attn.linears.3.weight" in names
    assert set(engine.param_buffers[sid + 1]) == {n for n, _ in engine.module.get_named_param(sid + 1)}
    with pytest.raises(Exception):
        build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.float32, GPT_VARIANT, 0, True)
    with pytest.raises(NotImplementedError):
        build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.float32, GPT_VARIANT, 2, True)
    loss = engine.train_batch()
    assert loss.shape == (1,) and engine.global_steps == 1
    assert all(b is None for b in engine.pipe_buffers[f"output_{sid}"])


def test_sigterm_and_launch_observer_belong_to_one_engine(hiplib):
    """SIGTERM (the preemption notice) stops the engine that installed the handler at its next batch with exit code
    13 (reference engine.py:98-111, 1096-1097) and leaves another engine of the process alone; a GEMM launch observer
    set on one engine sees that engine's launches only and does not switch the other's graph replay off."""
    import os
    import signal
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 1, 4, 1, 2, 4, 64
    prev = signal.getsignal(signal.SIGTERM)
    try:
        a, _ = build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.bfloat16, GPT_VARIANT, 1, True, install_signal_handler=True)
        b, _ = build(hid, heads, ffn, L, S, sid, mb, M, seq, torch.bfloat16, GPT_VARIANT, 1, True)
        seen = []
        a.set_gemm_hook(lambda desc, launch, stream: (seen.append(desc), launch()))
        b.train_batch()
        assert not seen
        a.train_batch()
        # per layer and micro-batch: own forward and redundant forward 4 products each, own backward 4 input
        # gradients and the grouped weight-gradient launch
        assert len(seen) == M * L * (4 + 4 + 5)
        a.set_gemm_hook(None)
        os.kill(os.getpid(), signal.SIGTERM)
        assert a.should_stop and not b.should_stop
        b.train_batch()
        with pytest.raises(SystemExit) as e:
            a.train_batch()
        assert e.value.code == 13
    finally:
        signal.signal(signal.SIGTERM, prev)


@pytest.mark.parametrize("hid,heads,fused", [(128, 4, True), (96, 3, False), (128, 1, True), (192, 2, False)],
                         ids=["head-width-32-pairs", "head-width-32-odd-heads", "head-width-128", "head-width-96"])
def test_bf16_stage_with_other_head_widths_matches_oracle(hiplib, hid, heads, fused):
    """A bf16 stage whose heads are 32 (the reference GPT-2 script's default, gpt2.py:212-214: the fused kernels take
    an even number of them in pairs, an odd number materialises the probabilities), 128 (fused) or 96 wide (not),
    with redundant forwards: outputs, input gradients and parameter gradients against the fp64 oracle at the bf16 bars, and the
    redundant forward's output bit-equal to the own forward of the same layers on the same input."""
    ffn, L, S, sid, mb, M, seq = 256, 2, 4, 1, 2, 4, 64
    dtype = torch.bfloat16
    engine, q = build(hid, heads, ffn, L, S, sid, mb, M, seq, dtype, GPT_VARIANT, 1, True)
    assert engine.module.func_buckets[sid][0].fused_attention(engine.ctx) == fused
    st, peer = oracle_for(engine, q, GPT_VARIANT, hid, heads, ffn, L, S, sid, M, 1, True)
    keep = {}
    with NoStep(engine):
        engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
        engine.train_batch()
    torch.cuda.synchronize()
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    rel_err.lowp = True
    for k in range(M):
        for s_ in (sid, sid + 1):
            want = bufs["out"][(s_, k)].detach().view(mb * seq, hid)
            assert rel_err(keep[f"output_{s_}"][k], want) < 2e-2 and max_err(keep[f"output_{s_}"][k], want) < 5e-2
        assert rel_err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].view(mb * seq, hid)) < 2e-2
    ref = st.named_grads(sid)
    for name, g in engine.module.get_named_grad(sid):
        assert rel_err(g, ref[name], grad_floor(ref)) < 2e-2, name
    # the shadow layers run as a stage of their own on the own outputs: same bits as the redundant forward
    specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
    model2 = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid + 1, dtype=dtype, device=DEV)
    ctx2 = model2.prepare_context([sid + 1], mb, seq)
    model2.allocate_stash(sid + 1, ctx2, 1)
    for k in range(M):
        normal = model2.forward(keep[f"output_{sid}"][k], sid + 1, slot=0, ctx=ctx2)
        torch.cuda.synchronize()
        assert torch.equal(normal, keep[f"output_{sid + 1}"][k]), k


def test_gradient_clipping_in_the_optimizer_step(hiplib):
    """``gradient_clipping`` of the DeepSpeed JSON (deepspeed/runtime/engine.py:1526-1531): with a bound far below the
    gradient norm the step equals the oracle stage's Adam step on gradients scaled by max_norm / (norm + 1e-6); the
    reported norm is the oracle's; with a bound far above it the weights equal the unclipped run bit for bit."""
    from oracle import adam as oadam
    rel_err.lowp = False
    hid, heads, ffn, L, S, sid, mb, M, seq = 128, 2, 256, 2, 4, 1, 2, 4, 64

    def run(clip):
        specs = [LayerSpec(TransformerLayer, hid, heads, ffn, **GPT_VARIANT) for _ in range(L * S)]
        model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=torch.float32, device=DEV)
        q = SeededActivationQueue((mb, seq, hid), torch.float32, M, stage_ids=[sid, sid + 1], seed=7, device=DEV)
        cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "gradient_clipping": clip,
               "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}}
        engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, activation_queue=q, install_signal_handler=False)
        return engine, q
    plain, _ = run(0.0)
    loose, _ = run(1e9)
    tight, q = run(1e-3)
    st, peer = oracle_for(tight, q, GPT_VARIANT, hid, heads, ffn, L, S, sid, M, 0, False, dtype=torch.float32)
    before = {k: v.clone() for k, v in tight.module.get_named_param(sid)}
    for e in (plain, loose, tight):
        e.train_batch()
    torch.cuda.synchronize()
    assert torch.equal(plain.module.stage_params[sid].master, loose.module.stage_params[sid].master)
    assert float(loose.grad_norm[1]) == 1.0
    # oracle: gradients of the batch, clipped, then the Adam step
    st.run_batch(peer, optimizer_step=False)
    names = list(st.named_grads(sid))
    grads = [st.named_grads(sid)[n].detach().numpy().astype(np.float32).copy() for n in names]
    norm, coef = oadam.clip_grad_norm(grads, 1e-3)
    assert coef < 0.1 and abs(float(tight.grad_norm[0]) - norm) < 1e-4 * norm
    got = dict(tight.module.get_named_param(sid))
    for n, g in zip(names, grads):
        if n.endswith("linears.1.bias"):
            continue    # key bias: the exact gradient is zero, Adam normalises rounding noise
        p0 = before[n].cpu().numpy().copy()
        ref, m_ref = p0.copy(), np.zeros_like(p0)
        oadam.adam_step(ref, g, m_ref, np.zeros_like(ref), 1)
        d, dr = got[n].cpu().numpy() - p0, ref - p0
        assert float(np.abs(d - dr).max()) < 2e-4, n       # movement against lr = 1e-3, as in the unclipped test
        # the first moment is (1 - beta1) x the CLIPPED gradient: the first step's movement alone would not tell
        sp = tight.module.stage_params[sid]
        m_got = sp.view(sp.exp_avg, n).cpu().numpy()
        assert float(np.abs(m_got - m_ref).max()) < 1e-4 * float(np.abs(m_ref).max()) + 1e-12, n
    assert not torch.equal(plain.module.stage_params[sid].exp_avg, tight.module.stage_params[sid].exp_avg)


def _decoder_stage(dtype, variant, dropout=0.0, dead_from=None, grad_mode="queue", heads=2):
    """Engine (stage 1 of 4, one DecoderLayer per stage, redundant forwards on) and oracle on the same weights and
    inputs drawn from U(0, 0.4): the memory sqrt(1 - x) of every layer stays real (the sublayers move the stream by
    a few hundredths at these weight scales)."""
    from bamboo_amd import DecoderLayer
    hid, ffn, S, sid, mb, M, seq = 128, 256, 4, 1, 2, 4, 64
    specs = [LayerSpec(DecoderLayer, hid, heads, ffn, dropout=dropout, **variant) for _ in range(S)]
    model = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid, dtype=dtype, device=DEV)
    q = SeededActivationQueue((mb, seq, hid), dtype, M, stage_ids=[sid, sid + 1], seed=7, grad_mode=grad_mode, device=DEV)
    g = torch.Generator().manual_seed(77)
    q.activations = [(0.4 * torch.rand(mb, seq, hid, generator=g)).to(dtype).to(DEV) for _ in range(M)]
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M, "bf16": {"enabled": dtype == torch.bfloat16}}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, redundancy_level=1, eager_recovery=True,
                                            activation_queue=q, install_signal_handler=False)
    ocfg = ol.TransformerCfg(hidden=hid, heads=heads, ffn=ffn, decoder=True, dropout=dropout, **variant)
    st = OracleStage(ocfg, list(range(S + 1)), sid, M, dtype=torch.float64, redundancy_level=1, eager=True)
    for s_ in list(st.params):
        sp = engine.module.stage_params[s_]
        named = sp.named(sp.compute)
        assert set(named) == set(st.named_params(s_))
        for key, t in st.named_params(s_).items():
            with torch.no_grad():
                t.copy_(named[key].double().cpu())
    acts = [a.double().cpu() for a in q.activations]
    if grad_mode == "queue":
        peer = OraclePeer(acts, M, grads={s_: [t.double().cpu() for t in gs] for s_, gs in q.grads.items()})
    else:
        peer = OraclePeer(acts, M, targets={s_: [t.double().cpu() for t in ts] for s_, ts in q.targets.items()})
    return engine, q, st, peer, (hid, mb, M, seq, sid)


@pytest.mark.parametrize("dtype,variant,heads", [(torch.float32, REFERENCE_VARIANT, 2), (torch.float32, GPT_VARIANT, 2),
                                                 (torch.bfloat16, GPT_VARIANT, 2), (torch.bfloat16, GPT_VARIANT, 4)],
                         ids=["fp32-script-variant", "fp32-gpt", "bf16-gpt", "bf16-gpt-head-width-32"])
def test_decoder_stage_matches_oracle_with_rc(hiplib, dtype, variant, heads):
    """A stage of the GPT-2 script's layers (DecoderLayerSimple, gpt2.py:20-34: self-attention, attention over
    sqrt(1 - x) of the layer input, feed-forward) with redundant forwards: own and redundant outputs, the gradient
    sent upstream (which also flows through the memory) and all 26 parameter gradients of the own layer against
    the fp64 oracle; the shadow layer's gradients stay zero.  The last case has the script's own head width (512 / 16 =
    32, gpt2.py:212-214): both attentions of the layer on the fused kernels, heads in pairs."""
    engine, q, st, peer, (hid, mb, M, seq, sid) = _decoder_stage(dtype, variant, heads=heads)
    if dtype == torch.bfloat16:
        assert engine.module.func_buckets[sid][0].fused_attention(engine.ctx)
    keep = {}
    with NoStep(engine):
        engine._clean_pipe_buffers = lambda: keep.update({k: list(v) for k, v in engine.pipe_buffers.items()})
        engine.train_batch()
    torch.cuda.synchronize()
    bufs, _ = st.run_batch(peer, optimizer_step=False)
    t_act, t_grad = (1e-5, 1e-4) if dtype == torch.float32 else (2e-2, 2e-2)
    rel_err.lowp = dtype == torch.bfloat16
    for k in range(M):
        for s_ in (sid, sid + 1):
            want = bufs["out"][(s_, k)].detach().view(mb * seq, hid)
            assert not torch.isnan(want).any()
            assert rel_err(keep[f"output_{s_}"][k], want) < t_act, (s_, k)
        assert rel_err(keep[f"input_grad_{sid}"][k], bufs["sent_grad"][(sid, k)].view(mb * seq, hid)) < t_grad, k
    ref = st.named_grads(sid)
    assert len(ref) == 26
    for name, g in engine.module.get_named_grad(sid):
        assert rel_err(g, ref[name], grad_floor(ref)) < t_grad, name
    for name, g in engine.module.get_named_grad(sid + 1):
        assert float(g.abs().max()) == 0.0
    # the redundant forward is bit-equal to the same layer run as a stage of its own on the same input
    from bamboo_amd import DecoderLayer
    heads, ffn, S = engine.module.func_buckets[sid][0].heads, engine.module.func_buckets[sid][0].ffn, engine.num_stages
    specs = [LayerSpec(DecoderLayer, hid, heads, ffn, **variant) for _ in range(S)]
    model2 = PipelineModule(specs, num_stages=S, partition_method="uniform", stage_id=sid + 1, dtype=dtype, device=DEV)
    ctx2 = model2.prepare_context([sid + 1], mb, seq)
    model2.allocate_stash(sid + 1, ctx2, 1)
    for k in range(M):
        normal = model2.forward(keep[f"output_{sid}"][k], sid + 1, slot=0, ctx=ctx2)
        torch.cuda.synchronize()
        assert torch.equal(normal, keep[f"output_{sid + 1}"][k]), k


@pytest.mark.parametrize("dtype,dropout", [(torch.float32, 0.0), (torch.bfloat16, 0.0), (torch.float32, 0.1)], ids=["fp32", "bf16", "fp32-dropout"])
def test_decoder_stage_failover_matches_oracle(hiplib, dtype, dropout):
    """The successor is lost at micro-batch 2: the promoted decoder layer's backward passes run from the stash of the
    redundant forwards (which left the activation derivative out: it is produced first), with dropout at the layer's
    six sites making the redundant forward's decisions again; gradients of both stages and the loss against the
    oracle's run of the same stream."""
    variant = dict(GPT_VARIANT)
    engine, q, st, peer, (hid, mb, M, seq, sid) = _decoder_stage(dtype, variant, dropout=dropout, dead_from=2, grad_mode="mse")
    true_grads = []
    for k in range(M):
        o1 = st.forward(peer.activations[k], sid, drop_id=(0, k)).detach().requires_grad_(True)
        o2 = st.forward(o1, sid + 1, drop_id=(0, k))
        (torch.nn.functional.mse_loss(o2, peer.targets[sid + 1][k]) / M).backward()
        true_grads.append(o1.grad)
    for s_ in st.params.values():
        for p in s_:
            for t in p.values():
                t.grad = None
    peer.targets = {sid + 1: peer.targets[sid + 1]}
    peer.grads = {sid: true_grads}
    peer.dead_from, peer.dead_stage = 2, sid
    st.run_batch(peer, optimizer_step=False)
    q.set_grads(sid, [g.view(mb, seq, hid) for g in true_grads])
    q.targets.pop(sid)
    orig_send = q.send_activation
    q.send_activation = lambda k, t, stage_id, stream=None: (q._check_alive(k, stage_id) if stage_id == sid
                                                              else orig_send(k, t, stage_id, stream=stream))
    q.preempt_successor(2, sid)
    with NoStep(engine):
        loss = engine.train_batch()
    assert engine.stage_ids == [sid, sid + 1]
    tg = 1e-4 if dtype == torch.float32 else 2e-2
    rel_err.lowp = dtype == torch.bfloat16
    for s_ in (sid, sid + 1):
        ref = st.named_grads(s_)
        for name, g in engine.module.get_named_grad(s_):
            assert rel_err(g, ref[name], grad_floor(ref)) < tg, (s_, name)
    assert abs(float(loss) - float(peer.loss) / M) < tg * max(1.0, float(peer.loss) / M)


def test_gpt2_script_layers_taken_over_run_as_the_last_stage(hiplib):
    """The GPT-2 script's own layer list (``GPT2Simple.join_layers``, gpt2.py:149-150: DecoderLayerSimple modules, the
    final LayerNorm, ``x.sum(-1)``) with ``nn.MSELoss()``, handed over as it is: the last stage (one decoder layer,
    norm, sum) on the HIP kernels against torch autograd on the modules themselves (fp32), inputs in (0, 0.4)."""
    from tests.reference_shapes import RefDecoderLayer, RefLayerNorm
    hid, heads, ffn, mb, M, seq = 128, 2, 256, 2, 4, 64
    torch.manual_seed(13)
    mods = [RefDecoderLayer(hid, heads, ffn, 0.0) for _ in range(2)] + [RefLayerNorm(hid)]
    with torch.no_grad():
        for m in mods:
            for prm in m.parameters():
                prm.add_(0.02 * torch.randn_like(prm))
    layers = mods + [lambda x: x.sum(-1)]
    g = torch.Generator().manual_seed(14)
    labels = [torch.randn(mb, seq, generator=g) for _ in range(M)]
    model = PipelineModule(layers, num_stages=2, partition_method="custom", custom_partitions=[0, 1, 4], stage_id=1,
                           loss_fn=torch.nn.MSELoss(), dtype=torch.float32, device=DEV)
    q = SeededActivationQueue((mb, seq, hid), torch.float32, M, stage_ids=[1], seed=5, device=DEV)
    q.activations = [(0.4 * torch.rand(mb, seq, hid, generator=g)).to(DEV) for _ in range(M)]
    cfg = {"train_micro_batch_size_per_gpu": mb, "gradient_accumulation_steps": M}
    engine, _, _, _ = bamboo_amd.initialize(model=model, config=cfg, activation_queue=q, install_signal_handler=False,
                                            training_data=[(torch.zeros(1), y) for y in labels])
    with NoStep(engine):
        loss = engine.train_batch()
    torch.cuda.synchronize()
    total, xgrads = 0.0, []
    for k in range(M):
        x = q.activations[k].cpu().clone().requires_grad_(True)
        l = torch.nn.functional.mse_loss(layers[3](mods[2](mods[1](x))), labels[k])
        (l / M).backward()
        total += float(l)
        xgrads.append(x.grad)
    rel_err.lowp = False
    assert abs(float(loss) - total / M) < 1e-5 * total / M
    ref = {f"{li}.{n}": p.grad for li in (1, 2) for n, p in mods[li].named_parameters()}
    got = dict(engine.module.get_named_grad(1))
    assert set(got) == set(ref)
    floor = grad_floor(ref)
    for name, gr in got.items():
        assert rel_err(gr, ref[name], floor) < 1e-4, name
    for k in range(M):
        assert rel_err(q.sent_grads[(1, k)], xgrads[k].view(mb * seq, hid)) < 1e-4
