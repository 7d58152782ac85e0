"""Layers of the reference's scripts handed to PipelineModule as they are (nn.Module instances, LayerSpec of module
classes, the x.sum(-1) callable): recognised by their parameters, replaced by native layers, weights taken over; and
the order / layout in which a layer's state travels (state_dict order of the reference module).  CPU only: building
the arenas runs no kernel in fp32."""
import pytest
import torch

from bamboo_amd import (BottleNeck, DecoderLayer, FinalLayerNorm, LayerSpec, MSELoss, PipelineError, PipelineModule, SumLast,
                        TransformerLayer)
from tests.reference_shapes import RefBottleNeck, RefDecoderLayer, RefEncoderLayer, RefLayerNorm


def encoder_script_layers(n=4, d=32, h=4, ff=64, p=0.0):
    """The layer list of the reference's transformer script (transformer.py:246-250): the encoder's layers, its
    final norm, and the sum over the hidden dimension."""
    torch.manual_seed(0)
    layers = [RefEncoderLayer(d, h, ff, p) for _ in range(n)]
    return layers + [RefLayerNorm(d), lambda x: x.sum(-1)]


def test_script_layer_list_is_taken_over():
    layers = encoder_script_layers()
    with torch.no_grad():
        for m in layers[:-1]:
            for prm in m.parameters():
                prm.add_(0.01 * torch.randn_like(prm))
    model = PipelineModule(layers, num_stages=2, loss_fn=torch.nn.MSELoss(), partition_method="uniform", stage_id=1,
                           dtype=torch.float32, device="cpu")
    assert isinstance(model.loss_fn, MSELoss)
    built = model.func_buckets[1]
    assert [type(b) for b in built] == [TransformerLayer, FinalLayerNorm, SumLast]
    assert (built[0].hidden, built[0].heads, built[0].ffn, built[0].activation, built[0].ln, built[0].mask) == (32, 4, 64, "relu", "annotated", "none")
    assert built[2].hidden == 32 and built[2].out_features == 1
    # weights: every parameter of the modules is in the arena under the reference's key "{layer_idx}.{name}"
    sp = model.stage_params[1]
    named = sp.named(sp.master)
    for li in (3, 4):
        for name, prm in layers[li].named_parameters():
            assert torch.equal(named[f"{li}.{name}"], prm.detach()), (li, name)
    assert set(named) == {f"{li}.{n}" for li in (3, 4) for n, _ in layers[li].named_parameters()}
    # the state of a layer travels in the module's own state_dict order
    assert list(model.layer_state_dict(3)) == list(layers[3].state_dict())
    assert list(model.layer_state_dict(4)) == list(layers[4].state_dict())
    assert list(model.layer_state_dict(5)) == []


def test_parameter_partitioning_counts_module_parameters():
    layers = encoder_script_layers(n=6)
    model = PipelineModule(layers, num_stages=3, partition_method="parameters", stage_id=0, dtype=torch.float32, device="cpu")
    assert model._count_layer_params()[:6] == [sum(p.numel() for p in layers[0].parameters())] * 6
    assert model._count_layer_params()[6:] == [64, 0]
    assert model.parts[0] == 0 and model.parts[-1] == 8 and model.parts == sorted(model.parts)


def test_layerspec_of_a_module_class_and_a_stage_that_opens_with_the_callable():
    torch.manual_seed(1)
    specs = [LayerSpec(RefEncoderLayer, 32, 4, 64, 0.0), LayerSpec(RefLayerNorm, 32), lambda x: x.sum(-1)]
    model = PipelineModule(specs, num_stages=2, partition_method="custom", custom_partitions=[0, 2, 3], stage_id=1,
                           dtype=torch.float32, device="cpu")
    (tail,) = model.func_buckets[1]
    assert isinstance(tail, SumLast) and tail.hidden == 32        # width taken from the layer in front of the stage


def test_what_is_not_recognised_is_refused():
    with pytest.raises(PipelineError, match="not one of the layers"):
        PipelineModule([torch.nn.Linear(8, 8)], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
    with pytest.raises(PipelineError, match="bare callable"):
        PipelineModule([RefEncoderLayer(32, 4, 64, 0.0), lambda x: x * 2], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
    # dropout: the module's probability in training mode, none in eval() mode; mixed probabilities are refused
    taken = PipelineModule([RefEncoderLayer(32, 4, 64, 0.1)], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu").func_buckets[0][0]
    assert isinstance(taken, TransformerLayer) and abs(taken.dropout - 0.1) < 1e-7 and taken.layer_idx == 0
    m = RefEncoderLayer(32, 4, 64, 0.1).eval()
    assert PipelineModule([m], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu").func_buckets[0][0].dropout == 0.0
    mixed = RefEncoderLayer(32, 4, 64, 0.1)
    mixed.feed_forward.dropout.p = 0.3
    with pytest.raises(PipelineError, match="different dropout"):
        PipelineModule([mixed], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
    with pytest.raises(PipelineError, match="MSELoss"):
        PipelineModule([m], num_stages=1, stage_id=0, loss_fn=torch.nn.L1Loss(), dtype=torch.float32, device="cpu")


def test_bottleneck_module_is_taken_over_with_layouts_and_running_statistics():
    torch.manual_seed(2)
    ref = RefBottleNeck(64, 16)
    with torch.no_grad():
        ref.residual_function[4].running_mean.add_(0.5)
    model = PipelineModule([ref, RefBottleNeck(64, 16)], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
    blk = model.func_buckets[0][0]
    assert isinstance(blk, BottleNeck) and (blk.cin, blk.cmid, blk.h) == (64, 16, None)
    sd = model.layer_state_dict(0)
    ref_params = dict(ref.named_parameters())
    assert list(sd) == [k for k in ref.state_dict() if k in ref_params]       # parameters in registration order
    for k, v in sd.items():
        assert v.shape == ref_params[k].shape and torch.equal(v, ref_params[k].detach()), k     # [O, I, kh, kw] on the wire
    # in the arena the 3x3 weight is tap-major
    sp = model.stage_params[0]
    w3 = sp.view(sp.master, "0.residual_function.3.weight")
    assert w3.shape == (16, 3, 3, 16) and torch.equal(w3.permute(0, 3, 1, 2), ref_params["residual_function.3.weight"].detach())
    # a tensor in the reference's layout goes back into the arena through the inverse conversion
    new = torch.randn(16, 16, 3, 3)
    model.load_layer_tensor(0, "residual_function.3.weight", new)
    assert torch.equal(model.layer_state_dict(0)["residual_function.3.weight"], new)
    assert float(blk._running("cpu")[4][0][0]) == 0.5


def test_downsampling_bottleneck_module_is_taken_over_with_its_shortcut():
    """A block with the projection shortcut (resnet.py:68-72): stride read off the 3x3 convolution, the shortcut's
    parameters follow the residual function's in the reference's registration order, its BatchNorm statistics come
    along; the partition by parameter count sees the extra parameters."""
    torch.manual_seed(3)
    ref = RefBottleNeck(64, 32, stride=2)
    with torch.no_grad():
        ref.shortcut[1].running_var.mul_(3.0)
    model = PipelineModule([ref, RefBottleNeck(128, 32)], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
    blk, plain = model.func_buckets[0]
    assert (blk.cin, blk.cmid, blk.cout, blk.stride, blk.projection) == (64, 32, 128, 2, True)
    assert (plain.stride, plain.projection, plain.feature_dim, plain.out_features) == (1, False, 128, 128)
    assert blk.out_seq(64) == 16 and blk.out_seq(49) == 16 and plain.out_seq(49) == 49
    sd = model.layer_state_dict(0)
    ref_params = dict(ref.named_parameters())
    assert list(sd) == [k for k in ref.state_dict() if k in ref_params]
    assert list(sd)[-3:] == ["shortcut.0.weight", "shortcut.1.weight", "shortcut.1.bias"]
    for k, v in sd.items():
        assert v.shape == ref_params[k].shape and torch.equal(v, ref_params[k].detach()), k
    assert float(blk._running("cpu")["shortcut"][1][0]) == 3.0
    assert blk.num_params() == sum(p.numel() for p in ref.parameters())


def test_bottleneck_whose_shortcut_contradicts_its_shape_is_refused():
    ref = RefBottleNeck(64, 16)                      # identity shortcut ...
    ref.residual_function[3].stride = (2, 2)         # ... but a stride: the reference would have built a projection
    with pytest.raises(PipelineError, match="projection shortcut"):
        PipelineModule([ref], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")


def test_seed_layers_gives_the_owner_and_the_shadow_the_same_weights():
    """``seed_layers=True`` (reference module.py:270-274): every LayerSpec is built under ``base_seed + layer_idx``, so the
    process that owns stage 2 and the one that shadows it start from equal weights whatever the ambient generator
    holds; auxiliary builds (parameter counting for the partition, widths, host mirrors) leave the generators alone;
    a ``seed_fn`` is called with the same seeds."""
    specs = lambda: [LayerSpec(RefEncoderLayer, 32, 4, 64, 0.0) for _ in range(6)] + [LayerSpec(RefLayerNorm, 32), lambda x: x.sum(-1)]
    kw = dict(num_stages=4, partition_method="parameters", dtype=torch.float32, device="cpu", seed_layers=True, base_seed=77)
    torch.manual_seed(5)
    owner = PipelineModule(specs(), stage_id=2, **kw)
    torch.manual_seed(6)                                     # another process: another ambient state
    torch.randn(17)
    pred = PipelineModule(specs(), stage_id=1, **kw)
    state = torch.get_rng_state()
    pred.allocate_param(2, {})                               # host mirrors: shapes only
    pred._count_layer_params()
    assert torch.equal(torch.get_rng_state(), state)
    pred.build_layers(2)                                     # the shadow stage
    a, b = owner.stage_params[2], pred.stage_params[2]
    assert list(a.index) == list(b.index) and a.numel > 0
    assert torch.equal(a.master, b.master)
    # the weights are those of a module built under that seed
    first = owner.parts[2]
    torch.manual_seed(77 + first)
    ref = RefEncoderLayer(32, 4, 64, 0.0)
    named = a.named(a.master)
    for name, prm in ref.named_parameters():
        assert torch.equal(named[f"{first}.{name}"], prm.detach()), name
    # without seed_layers the ambient generator decides (the reference's behaviour too)
    kw2 = dict(kw, seed_layers=False)
    torch.manual_seed(5)
    o2 = PipelineModule(specs(), stage_id=2, **kw2)
    torch.manual_seed(6)
    p2 = PipelineModule(specs(), stage_id=1, **kw2)
    p2.build_layers(2)
    assert not torch.equal(o2.stage_params[2].master, p2.stage_params[2].master)
    # seed_fn sees base_seed + layer_idx of every layer it builds for real, in order
    seen = []
    PipelineModule(specs(), stage_id=3, seed_fn=lambda s: (seen.append(s), torch.manual_seed(s)), **kw)
    assert seen == [77 + i for i in range(owner.parts[3], owner.parts[4]) if i < 7]


def test_gpt2_script_layer_list_is_taken_over():
    """The layer list of the reference's GPT-2 script (``GPT2Simple.join_layers``, gpt2.py:149-150: decoder layers, the
    final norm, the sum over the hidden dimension): every ``DecoderLayerSimple`` becomes a :class:`DecoderLayer` with
    the module's 26 parameters under the reference's keys, its state travels in the module's ``state_dict`` order,
    and the keys / values weights of the memory attention sit side by side in the arena (one product)."""
    torch.manual_seed(8)
    layers = [RefDecoderLayer(32, 4, 64, 0.1) for _ in range(4)] + [RefLayerNorm(32), lambda x: x.sum(-1)]
    model = PipelineModule(layers, num_stages=2, loss_fn=torch.nn.MSELoss(), partition_method="uniform", stage_id=0,
                           dtype=torch.float32, device="cpu")
    built = model.func_buckets[0]
    assert [type(b) for b in built] == [DecoderLayer] * 3
    assert (built[0].hidden, built[0].heads, built[0].ffn, built[0].activation, built[0].ln, built[0].mask) == (32, 4, 64, "relu", "annotated", "none")
    assert abs(built[0].dropout - 0.1) < 1e-7
    sp = model.stage_params[0]
    named = sp.named(sp.master)
    for li in range(3):
        want = dict(layers[li].named_parameters())
        assert len(want) == 26
        for name, prm in want.items():
            assert torch.equal(named[f"{li}.{name}"], prm.detach()), (li, name)
        assert list(model.layer_state_dict(li)) == list(layers[li].state_dict())
    kv = built[1].w["kv.weight"]
    assert kv.shape == (64, 32) and torch.equal(kv[:32], named["1.src_attn.linears.1.weight"]) and torch.equal(kv[32:], named["1.src_attn.linears.2.weight"])
    assert built[0].num_params() == sum(p.numel() for p in layers[0].parameters())
    # two attention modules that disagree on the heads are refused
    odd = RefDecoderLayer(32, 4, 64, 0.0)
    odd.src_attn.h = 2
    with pytest.raises(PipelineError, match="number of heads"):
        PipelineModule([odd], num_stages=1, stage_id=0, dtype=torch.float32, device="cpu")
