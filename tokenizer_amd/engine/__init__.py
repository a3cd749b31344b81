from .batch import EntryInfo, StepContext, StepEntry, build_context
from .engine import Engine, Model, load_model, random_model, resolve_dtype
from .generate import (Control, GenerateParams, Generated, SampleCursor, Sampled, StopHold, StopReason,
                       load_eos_token_ids, parse_eos_token_ids)
from .scheduler import EngineStats, Failure, QueueFull, Scheduler, SchedulerConfig
from .stream import StreamDecoder
from .api import generate, generate_with, greedy_tokens

__all__ = ["EntryInfo", "StepContext", "StepEntry", "build_context", "Engine", "Model", "load_model",
           "random_model", "resolve_dtype", "Control", "GenerateParams", "Generated", "SampleCursor", "Sampled",
           "StopHold", "StopReason", "load_eos_token_ids", "parse_eos_token_ids", "EngineStats", "Failure",
           "QueueFull", "Scheduler", "SchedulerConfig", "StreamDecoder", "generate", "generate_with",
           "greedy_tokens"]
