"""Taking over the layers of the reference's model scripts.

The reference's ``PipelineModule`` accepts ``nn.Module`` instances, ``LayerSpec`` of module classes and bare
callables in its layer list (deepspeed/runtime/pipe/module.py:281-318).  This engine runs hand-written kernels
with explicit backward passes, so it cannot execute an arbitrary module; what it can do is recognise the layers
the reference's own scripts are made of -- by the names and shapes of their parameters, not by their class, so a
script's local copy of the class is recognised too -- build the native layer that computes the same function, and
take the module's weights into the stage's arenas:

  ``EncoderLayer``   (DeepSpeedExamples/pipeline_parallelism/transformer.py:161-172;
                     ``EncoderLayerSimple``, bert.py:20-31: same parameters, same function)   -> :class:`TransformerLayer`
  ``DecoderLayerSimple`` (DeepSpeedExamples/pipeline_parallelism/gpt2.py:20-34)        -> :class:`DecoderLayer`
  ``LayerNorm``      (transformer.py:77-88, the ``encoder.norm`` of :181,250)          -> :class:`FinalLayerNorm`
  ``lambda x: x.sum(-1)`` (transformer.py:250)                                        -> :class:`SumLast`
  ``BottleNeck``     (DeepSpeedExamples/pipeline_parallelism/resnet.py:49-75)          -> :class:`BottleNeck`
  ``nn.MSELoss()``   (transformer.py:264, as ``loss_fn``)                              -> :class:`MSELoss`

Anything else is refused with an error that says what was found: there is no autograd fallback.
"""
import torch

from .layers import BottleNeck, DecoderLayer, FinalLayerNorm, MSELoss, SumLast, TransformerLayer


class AdoptionError(Exception):
    pass


def _dropout_probabilities(module):
    return sorted({float(m.p) for m in module.modules() if isinstance(m, torch.nn.Dropout)})


def _is_sum_last(fn):
    """Behavioural check of a bare callable: does it reduce the last dimension by summation?"""
    g = torch.Generator().manual_seed(0)
    for shape in ((2, 3, 8), (1, 5, 16)):
        x = torch.randn(shape, generator=g, dtype=torch.float64)
        try:
            y = fn(x)
        except Exception:
            return False
        if not (isinstance(y, torch.Tensor) and y.shape == x.shape[:-1] and torch.allclose(y, x.sum(-1), rtol=1e-12, atol=1e-12)):
            return False
    return True


def adopt_layer(obj, training=True):
    """``(native layer, {parameter name: tensor in the reference's layout} or None)`` for a layer object of the
    reference's scripts.  ``training``: dropout probabilities count (a module in ``eval()`` mode applies none)."""
    if all(hasattr(obj, a) for a in ("forward", "backward", "param_specs")):
        return obj, None                                     # already native
    if not isinstance(obj, torch.nn.Module):
        if callable(obj) and _is_sum_last(obj):
            return SumLast(hidden=None), None
        raise AdoptionError(f"layer {obj!r} is neither a layer of this package nor one of the reference scripts' layers "
                            "(a bare callable is taken only if it computes x.sum(-1)); this engine has no autograd fallback")
    params = {n: p.detach() for n, p in obj.named_parameters()}
    names = set(params)
    drops = _dropout_probabilities(obj) if (training and obj.training) else []
    if names == set(TransformerLayer.REFERENCE_ORDER):
        hidden = params["sublayer.0.norm.a_2"].numel()
        ffn = params["feed_forward.w_1.weight"].shape[0]
        heads = getattr(getattr(obj, "self_attn", None), "h", None)
        if heads is None:
            raise AdoptionError("EncoderLayer-shaped module without self_attn.h (number of heads)")
        if len(drops) > 1:
            raise AdoptionError(f"EncoderLayer-shaped module with different dropout probabilities {drops}: the layer "
                                "takes one probability for its four dropout sites, as the reference's make_encoder sets them")
        eps = float(getattr(obj.sublayer[0].norm, "eps", 1e-6))
        layer = TransformerLayer(hidden, int(heads), ffn, activation="relu", ln="annotated", mask="none", ln_eps=eps,
                                 dropout=drops[0] if drops else 0.0)
        return layer, params
    if names == set(DecoderLayer.REFERENCE_ORDER):
        hidden = params["sublayer.0.norm.a_2"].numel()
        ffn = params["feed_forward.w_1.weight"].shape[0]
        heads = getattr(getattr(obj, "self_attn", None), "h", None)
        if heads is None or getattr(getattr(obj, "src_attn", None), "h", None) != heads:
            raise AdoptionError("DecoderLayerSimple-shaped module whose two attention modules do not state one number of heads (.h)")
        if len(drops) > 1:
            raise AdoptionError(f"DecoderLayerSimple-shaped module with different dropout probabilities {drops}: the layer "
                                "takes one probability for its six dropout sites")
        eps = float(getattr(obj.sublayer[0].norm, "eps", 1e-6))
        layer = DecoderLayer(hidden, int(heads), ffn, activation="relu", ln="annotated", mask="none", ln_eps=eps,
                             dropout=drops[0] if drops else 0.0)
        return layer, params
    if names in (set(BottleNeck.RESIDUAL_ORDER), set(BottleNeck.RESIDUAL_ORDER + BottleNeck.SHORTCUT_ORDER)):
        w0, conv3 = params["residual_function.0.weight"], obj.residual_function[3]
        stride = conv3.stride[0] if isinstance(conv3.stride, tuple) else int(conv3.stride)
        bn = obj.residual_function[1]
        layer = BottleNeck(w0.shape[1], w0.shape[0], stride=stride, height=None, width=None, bn_eps=float(bn.eps),
                           bn_momentum=float(bn.momentum))
        if layer.projection != ("shortcut.0.weight" in names):
            raise AdoptionError(f"BottleNeck-shaped module: stride {stride}, {w0.shape[1]} -> {4 * w0.shape[0]} channels "
                                f"{'needs' if layer.projection else 'cannot have'} a projection shortcut (resnet.py:68-72)")
        stats = lambda m: (m.running_mean.detach().clone(), m.running_var.detach().clone())
        layer.adopted_running = {i: stats(obj.residual_function[i]) for i in (1, 4, 7)}
        if layer.projection:
            sc = obj.shortcut[0]
            sc_stride = sc.stride[0] if isinstance(sc.stride, tuple) else int(sc.stride)
            if sc_stride != stride:
                raise AdoptionError(f"BottleNeck-shaped module: shortcut stride {sc_stride} differs from the 3x3 "
                                    f"convolution's {stride}")
            layer.adopted_running["shortcut"] = stats(obj.shortcut[1])
        return layer, params
    if names == {"a_2", "b_2"}:
        return FinalLayerNorm(params["a_2"].numel(), ln="annotated", ln_eps=float(getattr(obj, "eps", 1e-6))), params
    raise AdoptionError(f"module {type(obj).__name__} with parameters {sorted(names)[:6]}... is not one of the layers this "
                        "engine accelerates (EncoderLayer, DecoderLayerSimple, LayerNorm, BottleNeck of the reference's pipeline_parallelism scripts)")


def adopt_loss(loss_fn):
    if loss_fn is None or isinstance(loss_fn, MSELoss):
        return loss_fn
    if isinstance(loss_fn, torch.nn.MSELoss):
        if loss_fn.reduction != "mean":
            raise AdoptionError("nn.MSELoss is taken with reduction='mean' only")
        return MSELoss()
    raise AdoptionError(f"loss_fn {loss_fn!r}: only nn.MSELoss() (the reference scripts' loss) has a kernel here")
