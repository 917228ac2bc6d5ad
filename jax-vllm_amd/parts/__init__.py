from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)
from .model import DecoderModel, Layer, RunMemoryPlan
from .spec import (
    PagedCacheSpec,
    PagedTensorSpec,
    LayerMemory,
    LayerRun,
    LayerSpec,
    ModelSpec,
    PartSpec,
    StateSpec,
    StepContext,
    TensorSpec,
    build_part,
    is_replayable,
    kv_cache_spec,
    register_part,
)

__all__ = [
    "DecoderModel", "Layer", "RunMemoryPlan", "PagedCacheSpec", "PagedTensorSpec", "kv_cache_spec", "LayerMemory", "LayerRun", "LayerSpec", "ModelSpec",
    "PartSpec", "StateSpec", "StepContext", "TensorSpec", "build_part", "is_replayable", "register_part",
]
