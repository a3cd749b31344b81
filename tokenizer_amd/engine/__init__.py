from .batch import EntryInfo, StepContext, StepEntry, build_context
from .engine import Engine, Model, load_model, random_model, resolve_dtype

__all__ = ["EntryInfo", "StepContext", "StepEntry", "build_context", "Engine", "Model", "load_model",
           "random_model", "resolve_dtype"]
