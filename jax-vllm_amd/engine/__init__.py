from .entries import StepEntry
from .request import EngineStats, Request, SamplingParams, StepEvent
from .scheduler import ScheduledItem, Scheduler, SchedulerOutput

__all__ = ["EngineCore", "StepEntry", "Engine", "LLM", "add_request", "has_work", "make_driver", "step", "EngineStats",
           "Request", "SamplingParams", "StepEvent", "ScheduledItem", "Scheduler", "SchedulerOutput"]


def __getattr__(name):
    if name == "EngineCore":  # pulls in torch and the kernels
        from .core import EngineCore

        return EngineCore
    if name in ("Engine", "LLM", "add_request", "has_work", "make_driver", "step"):
        from . import llm

        return getattr(llm, name)
    raise AttributeError(name)
