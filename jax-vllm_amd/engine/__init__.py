from .core import EngineCore, StepEntry
from .llm import LLM, add_request, has_work, make_driver, step
from .request import EngineStats, Request, SamplingParams, StepEvent
from .scheduler import ScheduledItem, Scheduler, SchedulerOutput

__all__ = ["EngineCore", "StepEntry", "LLM", "add_request", "has_work", "make_driver", "step", "EngineStats",
           "Request", "SamplingParams", "StepEvent", "ScheduledItem", "Scheduler", "SchedulerOutput"]
