"""``deepspeed.pipe`` namespace of the reference (deepspeed/pipe/__init__.py:1)."""
from ..module import LayerSpec, PipelineModule, TiedLayerSpec

__all__ = ["PipelineModule", "LayerSpec", "TiedLayerSpec"]
