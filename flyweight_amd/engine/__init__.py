from .engine import EngineError, Model, Runtime
from .model import CacheView, CausalLM, declared_tensors, load_model, parse_dtype
from .scheduler import (EVENT_ERROR, EVENT_FINISHED, EVENT_PREFILL, EVENT_TOKEN, Request, Scheduler,
                        SchedulerError, StepPlan)
from .step import StepContext, StepEntry, StepError, Stepper

__all__ = ["EngineError", "Model", "Runtime", "CacheView", "CausalLM", "declared_tensors", "load_model",
           "parse_dtype", "EVENT_ERROR", "EVENT_FINISHED", "EVENT_PREFILL", "EVENT_TOKEN", "Request", "Scheduler",
           "SchedulerError", "StepPlan", "StepContext", "StepEntry", "StepError", "Stepper"]
