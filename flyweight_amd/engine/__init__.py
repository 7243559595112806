from .model import CacheView, CausalLM, declared_tensors, load_model, parse_dtype
from .step import StepContext, StepEntry, StepError, Stepper

__all__ = ["CacheView", "CausalLM", "declared_tensors", "load_model", "parse_dtype", "StepContext", "StepEntry",
           "StepError", "Stepper"]
