"""A whole pipeline on one GPU (one engine per stage, threads, LocalFabric): parity of the
failure-free run with the CPU oracle of the unpartitioned model, and the reference's three-party
failure protocol -- a middle stage is lost mid-batch, its predecessor replays its work from the
redundant forwards, its successor re-sends gradients -- checked bit for bit against the run in
which nothing fails, gradients first, then weights after several optimizer steps (which also
needs the shadow-weight refresh)."""
import pytest
import torch
import torch.nn.functional as F

from bamboo_amd import LayerSpec, MSELoss, TransformerLayer, schedule
from bamboo_amd.local_pipeline import LocalPipeline
from oracle import layers as ol
from oracle.stage import OracleStage

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
HID, HEADS, FFN, S, MB, M, SEQ = 128, 2, 256, 4, 2, 4, 64
VARIANT = dict(activation="gelu_tanh", ln="standard", mask="causal")


def make_data(dtype, seed=3):
    g = torch.Generator().manual_seed(seed)
    return [(torch.randn(MB, SEQ, HID, generator=g).to(dtype).to(DEV), torch.randn(MB, SEQ, HID, generator=g).to(dtype).to(DEV))
            for _ in range(M)]


def make_pipeline(dtype, layers_per_stage=1, eager=True, rc_stream=False, data=None):
    specs = [LayerSpec(TransformerLayer, HID, HEADS, FFN, **VARIANT) for _ in range(S * layers_per_stage)]
    cfg = {"train_micro_batch_size_per_gpu": MB, "gradient_accumulation_steps": M,
           "optimizer": {"type": "Adam", "params": {"lr": 1e-3}}, "bf16": {"enabled": dtype == torch.bfloat16}}
    return LocalPipeline(specs, S, cfg, (MB, SEQ, HID), dtype, data if data is not None else make_data(dtype), MSELoss(),
                         redundancy_level=1, eager_recovery=eager, rc_stream=rc_stream, device=DEV, timeout=60.0)


def freeze_optimizer(pipe):
    """Keep the gradients: OptimizerStep becomes a no-op on every engine."""
    for e in pipe.engines.values():
        e._INSTRUCTION_MAP = dict(e._INSTRUCTION_MAP)
        e._INSTRUCTION_MAP[schedule.OptimizerStep] = lambda self_: None


def all_grads(pipe):
    out = {}
    for sid in range(S):
        for name, g in pipe.engine_of(sid).module.get_named_grad(sid):
            out[name] = g.clone()
    return out


def all_weights(pipe):
    out = {}
    for sid in range(S):
        sp = pipe.engine_of(sid).module.stage_params[sid]
        for name, w in sp.named(sp.master).items():
            out[name] = w.clone()
    return out


def rel(got, ref, floor):
    got, ref = got.double().cpu(), ref.double().cpu()
    return float((got - ref).abs().max() / max(float(ref.abs().max()), floor))


def test_pipeline_matches_unpartitioned_oracle(hiplib):
    dtype = torch.float32
    data = make_data(dtype)
    pipe = make_pipeline(dtype, data=data)
    freeze_optimizer(pipe)
    loss = pipe.train_batch(sync_weights=False)
    torch.cuda.synchronize()
    # oracle: all layers as one stage, fp64, same weights, loss_k / M per micro-batch
    cfg = ol.TransformerCfg(hidden=HID, heads=HEADS, ffn=FFN, **VARIANT)
    st = OracleStage(cfg, [0, S], 0, M, dtype=torch.float64, redundancy_level=0, eager=False)
    for sid in range(S):
        sp = pipe.engines[sid].module.stage_params[sid]
        named = sp.named(sp.compute)
        for key, t in st.named_params(0).items():
            if key in named:
                with torch.no_grad():
                    t.copy_(named[key].double().cpu())
    total = 0.0
    for x, y in data:
        out = st.forward(x.double().cpu(), 0, None)
        l = F.mse_loss(out, y.double().cpu())
        (l / M).backward()
        total += float(l.detach())
    assert abs(float(loss) - total / M) < 1e-5 * abs(total / M)
    ref = st.named_grads(0)
    floor = 1e-3 * max(float(g.abs().max()) for g in ref.values())
    got = all_grads(pipe)
    assert set(got) == set(ref)
    for name, g in got.items():
        assert rel(g, ref[name], floor) < 1e-4, name


@pytest.mark.parametrize("dead_from", [0, 2, 3])
@pytest.mark.parametrize("victim", [1, 2])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["fp32", "bf16"])
def test_lost_stage_is_recovered_bit_exact(hiplib, dtype, victim, dead_from):
    data = make_data(dtype)
    good = make_pipeline(dtype, data=data)
    freeze_optimizer(good)
    loss_good = good.train_batch(sync_weights=False)
    ref = all_grads(good)

    pipe = make_pipeline(dtype, data=data)
    freeze_optimizer(pipe)
    pipe.kill(victim, at_micro_batch=dead_from)
    loss = pipe.train_batch(sync_weights=False)
    torch.cuda.synchronize()
    assert pipe.lost == [victim]
    pred, succ = pipe.engines[victim - 1], pipe.engines[victim + 1]
    assert pred.stage_ids == [victim - 1, victim] and pred.r_stage_ids == []
    assert pred.last_failover["failed_step"] <= pred.last_failover["step"]
    assert float(loss) == float(loss_good)
    got = all_grads(pipe)
    for name, g in ref.items():
        assert torch.equal(got[name], g), name
    # the stage after the lost one either noticed (and switched streams) or had finished with it
    if succ.last_failover is not None:
        assert succ.last_failover["failed_step"] == pred.last_failover["failed_step"]
        assert succ._prev_failover == (0, 0)
    if dead_from == 0:
        assert succ.last_failover is not None     # it was waiting for the first activation
    # the next batch runs on three engines
    loss2 = pipe.train_batch(sync_weights=False)
    loss2_good = good.train_batch(sync_weights=False)
    assert float(loss2) == float(loss2_good)      # same weights (no step): same loss, gradients doubled
    got2, ref2 = all_grads(pipe), all_grads(good)
    for name, g in ref2.items():
        assert torch.equal(got2[name], g), name


@pytest.mark.parametrize("dead_from", [0, 1])
@pytest.mark.parametrize("victim", [1, 2])
def test_lazy_pipeline_notices_a_loss_through_its_pings(hiplib, victim, dead_from):
    """Lazy recovery (no redundant forwards, one-element pings on silent steps): a stage lost at its first
    micro-batches is noticed by its successor through a receive-ping (PrevStageException -- the successor keeps
    its own stream and re-sends gradients) and by its predecessor through a send (NextStageException -- it
    promotes the shadow stage from its host mirrors).  Gradients and loss equal the failure-free run bit for bit."""
    dtype = torch.float32
    data = make_data(dtype)
    good = make_pipeline(dtype, data=data, eager=False)
    freeze_optimizer(good)
    loss_good = good.train_batch(sync_weights=False)
    ref = all_grads(good)
    pipe = make_pipeline(dtype, data=data, eager=False)
    freeze_optimizer(pipe)
    pipe.kill(victim, at_micro_batch=dead_from)
    loss = pipe.train_batch(sync_weights=False)
    torch.cuda.synchronize()
    assert pipe.lost == [victim]
    pred, succ = pipe.engines[victim - 1], pipe.engines[victim + 1]
    assert pred.stage_ids == [victim - 1, victim] and succ.stage_ids == [victim + 1]
    assert succ.last_failover is not None and succ.last_failover.get("role") == "successor of the lost stage"
    assert float(loss) == float(loss_good)
    got = all_grads(pipe)
    for name, g in ref.items():
        assert torch.equal(got[name], g), name


@pytest.mark.parametrize("eager", [True, False], ids=["eager", "lazy"])
@pytest.mark.parametrize("rc_stream", [False, True], ids=["one-stream", "rc-stream"])
def test_training_through_a_failure_equals_training_without(hiplib, rc_stream, eager):
    """Three optimizer steps; the victim disappears in the second batch.  Equal weights at the end
    need fresh shadow weights AND moments at the moment of promotion (SendWeights/RecvWeights)."""
    dtype = torch.bfloat16
    data = make_data(dtype)
    good = make_pipeline(dtype, data=data, rc_stream=rc_stream, eager=eager)
    pipe = make_pipeline(dtype, data=data, rc_stream=rc_stream, eager=eager)
    losses_good, losses = [], []
    for b in range(3):
        losses_good.append(float(good.train_batch()))
    for b in range(3):
        if b == 1:
            pipe.kill(2, at_micro_batch=1)
        losses.append(float(pipe.train_batch()))
    torch.cuda.synchronize()
    assert losses == losses_good
    assert losses[2] != losses[0]                  # the optimizer did move the weights
    w, w_good = all_weights(pipe), all_weights(good)
    for name, t in w_good.items():
        assert torch.equal(w[name], t), name
    # redundant forwards are useful only with fresh shadows: stage 0 shadows stage 1
    e0 = pipe.engines[0]
    sp_real = pipe.engine_of(1).module.stage_params[1]
    if eager:
        sp_shadow = e0.module.stage_params[1]
        assert torch.equal(sp_shadow.master, sp_real.master) and torch.equal(sp_shadow.exp_avg_sq, sp_real.exp_avg_sq)
    else:
        for name, w in sp_real.named(sp_real.master).items():
            assert torch.equal(e0.param_buffers[1][name], w.cpu()), name


def test_without_refresh_the_shadow_goes_stale(hiplib):
    pipe = make_pipeline(torch.float32)
    pipe.train_batch(sync_weights=False)
    e0 = pipe.engines[0]
    assert not torch.equal(e0.module.stage_params[1].master, pipe.engines[1].module.stage_params[1].master)
    pipe.sync_shadow_weights()
    assert torch.equal(e0.module.stage_params[1].master, pipe.engines[1].module.stage_params[1].master)


def test_layers_travel_between_engines_and_through_checkpoints(hiplib, tmp_path):
    """send_layers / recv_layers (two flat tensors) and layer_XX-model_states.pt files."""
    dtype = torch.bfloat16
    a = make_pipeline(dtype, layers_per_stage=2)
    a.train_batch()                                        # moments and weights away from their initial values
    src, dst = a.engines[1], a.engines[0]                  # engine 0 holds shadow copies of layers 2 and 3
    idxs = [2, 3]
    state = src.get_layer_state(idxs)
    lt, ot = src.send_layers(0, idxs, state)
    n = sum(v.numel() for v in state[2][0].values()) + sum(v.numel() for v in state[3][0].values())
    assert lt.numel() == n and ot.numel() == 2 * n and lt.dtype == torch.float32
    sp_dst, sp_src = dst.module.stage_params[1], src.module.stage_params[1]
    sp_dst.master.zero_(); sp_dst.exp_avg.zero_(); sp_dst.exp_avg_sq.zero_()
    dst.load_layer_state(dst.recv_layers(1, idxs))         # through the fabric mailbox
    assert torch.equal(sp_dst.master, sp_src.master) and torch.equal(sp_dst.exp_avg, sp_src.exp_avg)
    assert torch.equal(sp_dst.exp_avg_sq, sp_src.exp_avg_sq) and torch.equal(sp_dst.compute, sp_src.compute)
    # checkpoint files, one per layer, loadable with weights_only
    src.module.save_state_dict(str(tmp_path))
    assert sorted(p.name for p in tmp_path.iterdir()) == ["layer_02-model_states.pt", "layer_03-model_states.pt"]
    sd = torch.load(str(tmp_path / "layer_02-model_states.pt"), weights_only=True)
    assert list(sd) == list(src.module.layer_state_dict(2))
    sp_dst.master.zero_()
    dst.module.load_state_dir(str(tmp_path), stage_id=1)
    assert torch.equal(sp_dst.master, sp_src.master) and torch.equal(sp_dst.compute, sp_src.compute)
    with pytest.raises(FileNotFoundError):
        dst.module.load_state_dir(str(tmp_path))           # stage 0's own layers were not saved
