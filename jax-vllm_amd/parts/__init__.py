from . import attention, block, embedding, mlp, norm, rotary  # noqa: F401  (register the built-in parts)
from .model import DecoderModel, Layer, RunMemoryPlan
from .spec import (
    KVCacheSpec,
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
    register_part,
)

__all__ = [
    "DecoderModel", "Layer", "RunMemoryPlan", "KVCacheSpec", "LayerMemory", "LayerRun", "LayerSpec", "ModelSpec",
    "PartSpec", "StateSpec", "StepContext", "TensorSpec", "build_part", "is_replayable", "register_part",
]
