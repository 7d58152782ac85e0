"""``PipelineModule`` / ``LayerSpec``: the layer list of a pipelined model and the layers this
process has materialised (its own stage and the stages it shadows).

Interface of ``deepspeed/runtime/pipe/module.py`` of the reference: constructor :95-106,
``build_layers(stage_id, buffer)`` :262-332, ``allocate_param`` :229-260,
``get_named_param`` :219-227, ``forward(x, stage_id)`` :516-574, ``_partition_layers``
:576-635.  Differences that follow from running on hand-written kernels instead of autograd:
layers are native layer objects (``bamboo_amd.layers``) with explicit forward/backward; the
parameters of a stage live in flat HBM arenas (fp32 master, fp32 gradient, compute-dtype copy)
and ``forward`` takes the stash slot that receives the activations of this micro-batch.
"""
import math
import os
import re
from collections import OrderedDict

import torch

from . import hip
from .layers import StageContext
from .utils import partition_balanced, partition_uniform


class PipelineError(Exception):
    """Errors related to the use of pipeline parallelism."""


class LayerSpec:
    """Delayed construction of a layer: ``LayerSpec(TransformerLayer, hidden=..., ...)``
    (reference module.py:25-69)."""

    def __init__(self, typename, *module_args, **module_kwargs):
        if not isinstance(typename, type):
            raise RuntimeError("LayerSpec expects a class")
        self.typename = typename
        self.module_args = module_args
        self.module_kwargs = module_kwargs

    def __repr__(self):
        from .schedule import call_to_str
        return call_to_str(self.typename.__name__, *self.module_args, **self.module_kwargs)

    def build(self, log=False):
        return self.typename(*self.module_args, **self.module_kwargs)


class TiedLayerSpec(LayerSpec):
    """Accepted for interface compatibility; tied layers are outside the accelerated path
    (the reference itself disables ReduceTiedGrads, schedule.py:283-285)."""

    def __init__(self, key, typename, *module_args, forward_fn=None, tied_weight_attr="weight", **module_kwargs):
        super().__init__(typename, *module_args, **module_kwargs)
        self.key, self.forward_fn, self.tied_weight_attr = key, forward_fn, tied_weight_attr


class MirrorBuffer(dict):
    """``{name: tensor}`` whose tensors are views of one flat tensor ``flat`` (set by whoever fills it)."""
    flat = None


def flat_mirror(numel, device="cpu"):
    """Zeroed fp32 tensor for a host mirror: page-locked where a GPU is present (transfers at the link's rate,
    asynchronous to the host), plain otherwise."""
    pin = torch.device(device).type == "cpu" and torch.cuda.is_available()
    return torch.zeros(numel, dtype=torch.float32, device=device, pin_memory=pin)


class StageParams:
    """Flat parameter arenas of one stage and the per-layer named views into them."""

    def __init__(self, layers, first_layer_idx, dtype, device):
        self.layers, self.dtype, self.device = layers, dtype, device
        self.index = OrderedDict()   # "{layer_idx}.{name}" -> (offset, shape)
        off = 0
        for li, layer in enumerate(layers):
            for name, shape in layer.param_specs().items():
                n = math.prod(shape)
                if n % 8:
                    raise PipelineError(f"parameter {name} of size {n} breaks the 16-byte arena alignment")
                self.index[f"{first_layer_idx + li}.{name}"] = (off, tuple(shape))
                off += n
        self.numel = off
        f32 = torch.float32
        self.master = torch.zeros(off, dtype=f32, device=device)
        self.grad = torch.zeros(off, dtype=f32, device=device)
        self.exp_avg = torch.zeros(off, dtype=f32, device=device)
        self.exp_avg_sq = torch.zeros(off, dtype=f32, device=device)
        self.compute = self.master if dtype == f32 else torch.zeros(off, dtype=dtype, device=device)
        self.first_layer_idx = first_layer_idx
        for li, layer in enumerate(layers):
            prefix = f"{first_layer_idx + li}."
            names = [k[len(prefix):] for k in self.index if k.startswith(prefix)]
            layer.layer_idx = first_layer_idx + li
            layer.bind({n: self.view(self.compute, prefix + n) for n in names},
                       {n: self.view(self.grad, prefix + n) for n in names})

    def view(self, arena, key):
        off, shape = self.index[key]
        return arena[off: off + math.prod(shape)].view(shape)

    def named(self, arena):
        return OrderedDict((k, self.view(arena, k)) for k in self.index)

    def init(self, base_seed):
        host = torch.zeros(self.numel, dtype=torch.float32)
        for li, layer in enumerate(self.layers):
            prefix = f"{self.first_layer_idx + li}."
            views = {k[len(prefix):]: host[o: o + math.prod(s)].view(s)
                     for k, (o, s) in self.index.items() if k.startswith(prefix)}
            layer.init_params(views, base_seed + self.first_layer_idx + li)
        self.master.copy_(host)
        self.refresh_compute()

    def refresh_compute(self):
        if self.compute is not self.master:
            hip.cast(self.master, self.compute)

    def load(self, named_tensors):
        """Copy ``{"{layer_idx}.{name}": tensor}`` into the master arena (missing keys are left).  Tensors in
        the reference's layout (4-D convolution weights) are converted by the layer's ``to_native``."""
        for k, t in named_tensors.items():
            if k in self.index:
                dst = self.view(self.master, k)
                layer = self.layers[int(k.split(".", 1)[0]) - self.first_layer_idx]
                if tuple(t.shape) != tuple(dst.shape) and hasattr(layer, "to_native"):
                    t = layer.to_native(k.split(".", 1)[1], t)
                dst.copy_(t.to(torch.float32).reshape(dst.shape))
        self.refresh_compute()


class PipelineModule:
    """Sequence of layers partitioned over ``num_stages`` pipeline stages.

    ``stage_id`` (keyword, or the ``pipe`` coordinate of ``PROJECT_PACTUM_COORDINATES`` /
    ``BAMBOO_STAGE_ID`` in the environment) says which stage this process executes; the
    reference obtains it from its rendezvous (module.py:150-170)."""

    def __init__(self, layers, num_stages=None, topology=None, loss_fn=None, seed_layers=False, seed_fn=None,
                 base_seed=1234, partition_method="parameters", custom_partitions=[],
                 activation_checkpoint_interval=0, activation_checkpoint_func=None, stage_id=None,
                 dtype=torch.float32, device=None):
        if num_stages is None and topology is None:
            raise RuntimeError("must provide num_stages or topology")
        if activation_checkpoint_interval < 0:
            raise ValueError("activation_checkpoint_interval must be >= 0")
        # Groups of this many layers keep only their input per micro-batch; the backward pass runs the
        # group's forward again (same kernels, same bits) into a work stash shared by all micro-batches
        # (reference: module.py:551-573; activation_checkpoint_func is accepted and unused: the stash is
        # explicit here, there is no autograd graph to cut).
        self.activation_checkpoint_interval = int(activation_checkpoint_interval)
        self.activation_checkpoint_func = activation_checkpoint_func
        self.num_stages = num_stages if num_stages is not None else topology.get_dim("pipe")
        if stage_id is None:
            stage_id = self._stage_from_env()
        if not 0 <= stage_id < self.num_stages:
            raise PipelineError(f"stage_id {stage_id} outside [0, {self.num_stages})")
        self.stage_id = stage_id
        from .adopt import AdoptionError, adopt_loss
        try:
            self.loss_fn = adopt_loss(loss_fn)
        except AdoptionError as e:
            raise PipelineError(str(e)) from None
        self.seed_layers, self.seed_fn, self.base_seed = seed_layers, seed_fn, base_seed
        self.micro_offset = 0
        self._layer_specs = list(layers)
        self._num_layers = len(self._layer_specs)
        self.partition_method = partition_method
        self.dtype = dtype
        self.device = torch.device(device if device is not None else "cuda:0")
        self.func_buckets = {}        # stage_id -> [layer objects]
        self.param_name_buckets = {}  # stage_id -> ["{layer_idx}.{name}"]
        self.stage_params = {}        # stage_id -> StageParams
        self._stash = {}              # stage_id -> [slot][layer] -> dict of views
        self._partition_layers(method=partition_method, partitions=custom_partitions)
        self.build_layers(self.stage_id)

    @staticmethod
    def _stage_from_env():
        if "BAMBOO_STAGE_ID" in os.environ:
            return int(os.environ["BAMBOO_STAGE_ID"])
        coords = os.environ.get("PROJECT_PACTUM_COORDINATES")
        if coords:
            import json
            c = json.loads(coords)
            first = c[0] if isinstance(c, list) and c and isinstance(c[0], (list, tuple)) else c
            return int(first[1])  # (dp_id, stage_id)
        return 0

    # ------------------------------------------------------------------ seeding
    def _seed_layer(self, layer_idx):
        """``seed_layers``: every layer is built under the seed ``base_seed + layer_idx`` (reference module.py:270-274;
        ``seed_fn`` if given, else random / numpy / torch as ``set_random_seed``, runtime/utils.py:51-61), so the
        process that owns a stage and the one that shadows it build the same weights from a ``LayerSpec``."""
        if not self.seed_layers:
            return
        seed = self.base_seed + layer_idx
        if self.seed_fn:
            self.seed_fn(seed)
        else:
            import random

            import numpy
            random.seed(seed)
            numpy.random.seed(seed)
            torch.manual_seed(seed)

    def _build_spec(self, layer_idx, auxiliary=False):
        """The layer object of ``_layer_specs[layer_idx]``.  ``auxiliary``: a build whose only purpose is to look at
        the layer (parameter count, width): the random generators are left as they were found."""
        spec = self._layer_specs[layer_idx]
        if not isinstance(spec, LayerSpec):
            return spec
        if not auxiliary:
            self._seed_layer(layer_idx)
            return spec.build()
        import random

        import numpy
        saved = (random.getstate(), numpy.random.get_state(), torch.get_rng_state())
        try:
            return spec.build()
        finally:
            random.setstate(saved[0])
            numpy.random.set_state(saved[1])
            torch.set_rng_state(saved[2])

    # ------------------------------------------------------------------ partitioning
    def _count_layer_params(self):
        """Trainable parameters per layer (reference module.py:337-360: modules count theirs, bare callables 0)."""
        counts = []
        for idx in range(len(self._layer_specs)):
            layer = self._build_spec(idx, auxiliary=True)
            if hasattr(layer, "num_params"):
                counts.append(layer.num_params())
            elif isinstance(layer, torch.nn.Module):
                counts.append(sum(p.numel() for p in layer.parameters() if p.requires_grad))
            else:
                counts.append(0)
        return counts

    def _find_layer_type(self, layername):
        rx = re.compile(layername, re.IGNORECASE)
        out = []
        for i, spec in enumerate(self._layer_specs):
            name = spec.typename.__name__ if isinstance(spec, LayerSpec) else type(spec).__name__
            if rx.search(name):
                out.append(i)
        return out

    def _partition_layers(self, method="uniform", partitions=[]):
        method = method.lower()
        if method == "custom":
            assert partitions, "Required customized partitions"
            self.parts = list(partitions)
        elif method == "uniform":
            self.parts = partition_uniform(self._num_layers, self.num_stages)
        elif method == "parameters":
            self.parts = partition_balanced(self._count_layer_params(), self.num_stages)
        elif method.startswith("type:"):
            weights = [0] * self._num_layers
            for i in self._find_layer_type(method.split(":")[1]):
                weights[i] = 1
            self.parts = partition_balanced(weights, self.num_stages)
        else:
            raise NotImplementedError(f"Partitioning method {method} not implemented.")
        if len(self.parts) != self.num_stages + 1 or self.parts[-1] != self._num_layers:
            raise PipelineError(f"partition {self.parts} does not cover {self._num_layers} layers in {self.num_stages} stages")
        self._local_start, self._local_stop = self.parts[self.stage_id], self.parts[self.stage_id + 1]

    # ------------------------------------------------------------------ building
    def _instantiate(self, stage_id, auxiliary=False):
        """Layer objects of a stage.  Layers of the reference's scripts (``nn.Module`` instances, ``LayerSpec`` of
        module classes, the ``x.sum(-1)`` callable; reference module.py:281-318) are replaced by the native layer
        that computes the same function; their weights are kept to be loaded into the arenas."""
        from .adopt import AdoptionError, adopt_layer
        built, weights = [], {}
        prev_features = None
        for li, spec in enumerate(self._layer_specs[self.parts[stage_id]: self.parts[stage_id + 1]]):
            if isinstance(spec, TiedLayerSpec):
                raise NotImplementedError("tied layers are not supported on the accelerated stage path")
            layer = self._build_spec(self.parts[stage_id] + li, auxiliary=auxiliary)
            try:
                layer, taken = adopt_layer(layer)
            except AdoptionError as e:
                raise PipelineError(str(e)) from None
            if getattr(layer, "hidden", 0) is None:      # a parameter-free layer takes its width from its predecessor
                if prev_features is None:
                    prev_features = self._features_before(self.parts[stage_id] + li)
                layer.hidden = prev_features
            prev_features = layer.out_features
            if taken:
                idx = self.parts[stage_id] + li
                weights.update({f"{idx}.{name}": t for name, t in taken.items()})
            built.append(layer)
        self._adopted_weights = weights
        return built

    def _features_before(self, layer_idx):
        """Output width of the layer in front of ``layer_idx`` (for a width-less layer that opens a stage)."""
        from .adopt import adopt_layer
        if layer_idx == 0:
            raise PipelineError("the first layer of the model must state its width")
        layer, _ = adopt_layer(self._build_spec(layer_idx - 1, auxiliary=True))
        return layer.out_features

    def build_layers(self, stage_id, buffer=None):
        """Materialise the layers of ``stage_id`` on the GPU (own stage, or a stage this process
        shadows).  ``buffer``: optional ``{"{layer_idx}.{name}": tensor}`` to copy weights from; where it is the
        mirror :meth:`allocate_param` made (one flat host tensor behind the named views), it goes over in one copy."""
        if stage_id in self.func_buckets:
            if buffer is not None:
                self.stage_params[stage_id].load(buffer)
            return self.param_name_buckets[stage_id]
        layers = self._instantiate(stage_id)
        sp = StageParams(layers, self.parts[stage_id], self.dtype, self.device)
        flat = getattr(buffer, "flat", None)
        if flat is not None and flat.numel() == sp.numel and not self._adopted_weights:
            sp.master.copy_(flat)                # every parameter comes from the mirror: no seeded initialisation
            sp.refresh_compute()
            buffer = None
        else:
            sp.init(self.base_seed)
        if self._adopted_weights:
            sp.load(self._adopted_weights)       # weights of the modules the layers were taken from
            self._adopted_weights = {}
        if buffer is not None:
            sp.load(buffer)
        self.func_buckets[stage_id] = layers
        self.stage_params[stage_id] = sp
        self.param_name_buckets[stage_id] = list(sp.index.keys())
        return self.param_name_buckets[stage_id]

    def allocate_param(self, stage_id, param_buffer, device="cpu"):
        """Zero mirrors of the parameters of ``stage_id`` (reference module.py:229-260): named tensors in
        ``param_buffer`` that are views of ONE flat tensor in the arena's order (``param_buffer.flat`` where the
        buffer is a :class:`MirrorBuffer`), page-locked when it lives on the host of a GPU process, so that a
        refresh and a promotion move it in a single transfer."""
        layers = self.func_buckets.get(stage_id)
        if not layers:
            layers = self._instantiate(stage_id, auxiliary=True)
            self._adopted_weights = {}           # only the shapes were wanted
        specs = [(f"{self.parts[stage_id] + li}.{name}", shape) for li, layer in enumerate(layers)
                 for name, shape in layer.param_specs().items()]
        flat = flat_mirror(sum(math.prod(shape) for _, shape in specs), device)
        off = 0
        for key, shape in specs:
            n = math.prod(shape)
            param_buffer[key] = flat[off: off + n].view(shape)
            off += n
        if isinstance(param_buffer, MirrorBuffer):
            param_buffer.flat = flat
        names = [key for key, _ in specs]
        self.param_name_buckets.setdefault(stage_id, names)
        return names

    # ------------------------------------------------------------------ layer state and checkpoints
    def _layer_home(self, layer_idx):
        """(stage parameters, layer object) of a built layer (global index)."""
        for sid, sp in self.stage_params.items():
            if self.parts[sid] <= layer_idx < self.parts[sid + 1]:
                return sp, sp.layers[layer_idx - self.parts[sid]]
        raise PipelineError(f"layer {layer_idx} is not built in this process")

    def layer_state_dict(self, layer_idx, arena="master"):
        """``state_dict`` of one layer (global index) as the reference module would give it: parameters in the
        reference's registration order and layout (convolution weights ``[O, I, kh, kw]``), fp32.  Views of the
        arena where the layouts agree, copies where they do not; ``arena`` may also name a moment arena
        (``exp_avg``, ``exp_avg_sq``), whose entries travel in the same order and layout."""
        sp, layer = self._layer_home(layer_idx)
        names = getattr(layer, "REFERENCE_ORDER", None) or tuple(layer.param_specs())
        if set(names) != set(layer.param_specs()):
            raise PipelineError(f"{type(layer).__name__}.REFERENCE_ORDER does not list the layer's parameters")
        to_ref = getattr(layer, "to_reference", lambda name, t: t)
        src = getattr(sp, arena)
        return OrderedDict((n, to_ref(n, sp.view(src, f"{layer_idx}.{n}"))) for n in names)

    def load_layer_tensor(self, layer_idx, name, tensor, arena="master"):
        """Inverse of :meth:`layer_state_dict` for one entry: a tensor in the reference's layout into the arena."""
        sp, layer = self._layer_home(layer_idx)
        dst = sp.view(getattr(sp, arena), f"{layer_idx}.{name}")
        if tuple(tensor.shape) != tuple(dst.shape) and hasattr(layer, "to_native"):
            tensor = layer.to_native(name, tensor)
        dst.copy_(tensor.to(torch.float32).reshape(dst.shape))

    def save_state_dict(self, save_dir, stage_id=None):
        """One ``layer_XX-model_states.pt`` per layer of the stage (reference module.py:804-826)."""
        import os

        from .wire import ckpt_layer_path
        os.makedirs(save_dir, exist_ok=True)
        sid = self.stage_id if stage_id is None else stage_id
        for idx in range(self.parts[sid], self.parts[sid + 1]):
            sd = OrderedDict((k, v.detach().clone().cpu()) for k, v in self.layer_state_dict(idx).items())
            torch.save(sd, ckpt_layer_path(save_dir, idx))

    def load_state_dir(self, load_dir, strict=True, stage_id=None):
        """Read the per-layer files back into the master arena (reference module.py:828-850)."""
        import os

        from .wire import ckpt_layer_path
        sid = self.stage_id if stage_id is None else stage_id
        sp = self.stage_params[sid]
        for idx in range(self.parts[sid], self.parts[sid + 1]):
            path = ckpt_layer_path(load_dir, idx)
            if not os.path.exists(path):
                if strict:
                    raise FileNotFoundError(path)
                continue
            sd = torch.load(path, map_location="cpu", weights_only=True)
            want = self.layer_state_dict(idx)
            if strict and set(sd) != set(want):
                raise PipelineError(f"{path}: keys {sorted(sd)} do not match the layer's {sorted(want)}")
            sp.load({f"{idx}.{k}": v for k, v in sd.items()})

    def get_named_param(self, stage_id):
        """(name, fp32 master view) pairs of a built stage."""
        sp = self.stage_params[stage_id]
        yield from sp.named(sp.master).items()

    def get_named_grad(self, stage_id):
        sp = self.stage_params[stage_id]
        yield from sp.named(sp.grad).items()

    def parameters(self):
        for sid in sorted(self.stage_params):
            for _, p in self.get_named_param(sid):
                yield p

    def num_layers(self, stage_id):
        return self.parts[stage_id + 1] - self.parts[stage_id]

    # ------------------------------------------------------------------ stash
    def _checkpoint_groups(self, stage_id):
        n, every = len(self.func_buckets[stage_id]), self.activation_checkpoint_interval
        return [(a, min(a + every, n)) for a in range(0, n, every)]

    def allocate_stash(self, stage_id, ctx, slots):
        """One arena holding, for every (slot, layer), the activations its backward needs.  With
        activation checkpointing: one such set of per-layer buffers for the whole stage (the work
        stash) plus, per slot, the input of every layer group and the stage output."""
        layers = self.func_buckets[stage_id]
        ckpt = self.activation_checkpoint_interval > 0
        seqs = self._stage_seqs(stage_id, ctx)
        plans, total = [], 0
        for li, layer in enumerate(layers):
            plan = []
            ctx.seq = seqs[li]
            for name, shape, dtype in layer.stash_specs(ctx):
                nbytes = math.prod(shape) * torch.empty((), dtype=dtype).element_size()
                plan.append((name, shape, dtype, total, nbytes))
                total += (nbytes + 255) // 256 * 256
            plans.append(plan)
        full_sets = 1 if ckpt else slots
        arena = torch.empty(total * full_sets, dtype=torch.uint8, device=self.device)
        table = []
        for s in range(full_sets):
            per_layer = []
            for plan in plans:
                views = {}
                for name, shape, dtype, off, nbytes in plan:
                    lo = s * total + off
                    views[name] = arena[lo: lo + nbytes].view(dtype).view(shape)
                per_layer.append(views)
            table.append(per_layer)
        nbytes_total = total * full_sets
        self._stash_arena = getattr(self, "_stash_arena", {})
        self._stash_arena[stage_id] = arena
        if ckpt:
            groups = self._checkpoint_groups(stage_id)
            es = torch.empty((), dtype=self.dtype).element_size()
            shapes = [(ctx.batch * seqs[a], layers[a].feature_dim) for a, _ in groups] + \
                     [(ctx.batch * seqs[-1], layers[-1].out_features)]
            sizes = [r * c for r, c in shapes]
            per_slot = sum((n * es + 255) // 256 * 256 for n in sizes)
            keep = torch.empty(per_slot * slots, dtype=torch.uint8, device=self.device)
            kept = []
            for s in range(slots):
                lo, bufs = s * per_slot, []
                for n, shape in zip(sizes, shapes):
                    bufs.append(keep[lo: lo + n * es].view(self.dtype).view(shape))
                    lo += (n * es + 255) // 256 * 256
                kept.append(bufs)          # [group inputs ..., stage output]
            self._kept = getattr(self, "_kept", {})
            self._kept[stage_id] = kept
            self._stash_arena[(stage_id, "kept")] = keep
            nbytes_total += per_slot * slots
            table = [table[0]] * slots     # every slot works in the one shared set
        self._stash[stage_id] = table
        ctx.seq = seqs[0]
        return nbytes_total

    def _stage_seqs(self, stage_id, ctx=None):
        """Positions per sample in front of every layer of a built stage and behind its last one (a down-sampling
        bottleneck changes them); set by :meth:`prepare_context`."""
        seqs = getattr(self, "stage_seq", {}).get(stage_id)
        if seqs is None:
            if ctx is None:
                raise PipelineError(f"stage {stage_id}: prepare_context has not seen this stage")
            seqs = self._chain_seqs(stage_id, ctx.seq)
        return seqs

    def _chain_seqs(self, stage_id, seq):
        seqs = [seq]
        for layer in self.func_buckets[stage_id]:
            out_seq = getattr(layer, "out_seq", None)
            seqs.append(out_seq(seqs[-1]) if out_seq is not None else seqs[-1])
        self.stage_seq = getattr(self, "stage_seq", {})
        self.stage_seq[stage_id] = seqs
        return seqs

    def stage_io_shapes(self, stage_id, batch):
        """((rows, features) of the stage's input, (rows, features) of its output) once its context is prepared."""
        seqs, layers = self._stage_seqs(stage_id), self.func_buckets[stage_id]
        return (batch * seqs[0], layers[0].feature_dim), (batch * seqs[-1], layers[-1].out_features)

    # ------------------------------------------------------------------ execution
    def forward(self, forward_input, stage_id, slot=0, ctx=None, defer=False, layers=None):
        """``defer``: leave out of the stash what only a backward pass reads and this forward can
        produce later from what it does keep (``backward(..., deferred=True)`` then produces it first).
        ``layers=(a, b)``: only layers a..b-1 of the stage (``forward_input`` is then the input of layer a):
        a forward cut into pieces runs the same kernels on the same operands as a whole one."""
        stage_layers = self.func_buckets.get(stage_id)
        if stage_layers is None:
            raise Exception(f"Unregistered stage id {stage_id}")
        x = forward_input
        stash = self._stash[stage_id][slot]
        seqs = self._stage_seqs(stage_id, ctx)
        if layers is not None:
            if self.activation_checkpoint_interval != 0:
                raise PipelineError("a forward cut into layer ranges needs the full stash (no activation checkpointing)")
            a, b = layers
            if a == 0:
                self.micro_offset += 1
            ctx.defer = defer
            for i in range(a, b):
                ctx.seq = seqs[i]
                x = stage_layers[i].forward(x, stash[i], ctx)
            ctx.defer = False
            return x
        layers = stage_layers
        self.micro_offset += 1
        if self.activation_checkpoint_interval == 0:
            ctx.defer = defer
            for i, (layer, st) in enumerate(zip(layers, stash)):
                ctx.seq = seqs[i]
                x = layer.forward(x, st, ctx)
            ctx.defer = False
            return x
        kept = self._kept[stage_id][slot]
        for g, (a, b) in enumerate(self._checkpoint_groups(stage_id)):
            hip.cast(x, kept[g], stream=ctx.stream)   # same-type copy: the group's input outlives the work stash
            x = kept[g]
            for i in range(a, b):
                ctx.seq = seqs[i]
                x = layers[i].forward(x, stash[i], ctx)
        hip.cast(x, kept[-1], stream=ctx.stream)
        return kept[-1]

    def backward(self, grad_output, grad_input, stage_id, slot=0, ctx=None, deferred=False):
        """Back-propagate through the layers of ``stage_id`` from the stash of ``slot``; parameter
        gradients accumulate in the stage's fp32 gradient arena, the input gradient is written to
        ``grad_input``.  ``deferred``: the stash was written by ``forward(..., defer=True)``."""
        layers = self.func_buckets[stage_id]
        ctx.deferred = deferred and self.activation_checkpoint_interval == 0
        stash = self._stash[stage_id][slot]
        seqs = self._stage_seqs(stage_id, ctx)
        n = len(layers)
        d = grad_output
        groups = self._checkpoint_groups(stage_id) if self.activation_checkpoint_interval > 0 else [(0, n)]
        for g in range(len(groups) - 1, -1, -1):
            a, b = groups[g]
            if self.activation_checkpoint_interval > 0:
                # run the group's forward again from its kept input; like a redundant forward it must not
                # update running statistics a second time
                was, ctx.redundant = ctx.redundant, True
                x = self._kept[stage_id][slot][g]
                for i in range(a, b):
                    ctx.seq = seqs[i]
                    x = layers[i].forward(x, stash[i], ctx)
                ctx.redundant = was
            presummed = False
            for i in range(b - 1, a - 1, -1):
                dst = grad_input if i == 0 else ctx.buf(f"d_layer{i % 2}", (ctx.batch * seqs[i], layers[i].feature_dim))
                # Inside a group the layer in front (whose stash is there) may ask for its incoming gradient to be
                # prepared by the kernel that writes it (a bottleneck: masked by its last ReLU, with the sums of its
                # last BatchNorm); a layer that does so says so, and the receiver is told.
                sink = None
                if i > a and hasattr(layers[i - 1], "grad_sink"):
                    ctx.seq = seqs[i - 1]
                    sink = layers[i - 1].grad_sink(stash[i - 1], ctx)
                ctx.seq = seqs[i]
                ctx.grad_sink, ctx.grad_sink_used, ctx.grad_presummed = sink, False, presummed
                layers[i].backward(d, dst, stash[i], ctx)
                presummed = ctx.grad_sink_used
                d = dst
            ctx.grad_sink, ctx.grad_sink_used, ctx.grad_presummed = None, False, False
        ctx.deferred = False
        return grad_input

    def prepare_context(self, stage_ids, batch, seq, stream=None, forward_only=False):
        """Execution context with scratch sized for the largest layer of the given stages
        (``forward_only``: a lane that only runs redundant forwards needs no backward scratch)."""
        ctx = StageContext(batch, seq, self.dtype, self.device, stream)
        ws = 0
        for n, sid in enumerate(stage_ids):
            # the first stage of the list takes ``seq`` positions per sample, each later one what its predecessor
            # in the list leaves (consecutive stages: own, then shadowed / absorbed)
            seqs = self._chain_seqs(sid, seq if n == 0 else self.stage_seq[stage_ids[n - 1]][-1])
            for li, layer in enumerate(self.func_buckets[sid]):
                ctx.seq = seqs[li]
                if hasattr(layer, "forward_scratch_specs"):
                    ctx.ensure_scratch(layer.forward_scratch_specs(ctx))
                ws = max(ws, layer.workspace_elems())
                if forward_only:
                    continue
                ctx.ensure_scratch(layer.scratch_specs(ctx))
                h = (ctx.rows, layer.feature_dim)
                ctx.ensure_scratch([("d_layer0", h, self.dtype), ("d_layer1", h, self.dtype)])
        ctx.ensure_workspace(ws)
        ctx.seq = seq
        return ctx
