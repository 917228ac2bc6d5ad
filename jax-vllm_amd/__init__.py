"""MI355X-native Qwen3 inference engine (import name ``jax_vllm_amd``)."""
from .config import ConfigError, EngineConfig
from .engine.request import EngineStats, Request, SamplingParams, StepEvent

__all__ = ["ConfigError", "EngineConfig", "Qwen3Config", "EngineStats", "Request", "SamplingParams", "StepEvent",
           "LLM", "make_driver", "add_request", "has_work", "step", "prewarm",
           "load_model", "write_random_model"]


def __getattr__(name):
    # the engine and the weight loader pull in torch and the kernels: loaded on first use
    if name in ("LLM", "make_driver", "add_request", "has_work", "step", "prewarm"):
        from .engine import llm

        return getattr(llm, name)
    if name == "Qwen3Config":
        from .models.qwen3 import Qwen3Config

        return Qwen3Config
    if name in ("load_model", "write_random_model", "random_model_on_device", "WeightsError"):
        from . import weights

        return getattr(weights, name)
    raise AttributeError(name)
