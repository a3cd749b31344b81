"""tokenizer_amd: a small inference engine for AMD MI355X (gfx950), built on hand-written HIP kernels.

The names follow the library of the reference's `qwen-infer` crate (qwen-infer/src/lib.rs:14-24):
`load_model`, `generate`, `generate_with`, `greedy_tokens`, `GenerateParams`, `Generated`, `StopReason`,
`Control`, `SampleCursor`, `greedy_token`, `sample_token`, `StreamDecoder`, `parse_eos_token_ids`,
`load_eos_token_ids`, and `Tokenizer.load_qwen`; beside them the engine's own `Engine` (one `step()` over a
mixed batch), `Scheduler`, `random_model` and `write_random_model`.
"""
from . import models  # noqa: F401  (registers the architectures)
from .config import ConfigError, Qwen2Config, load_config, register_architecture, registered_architectures
from .engine import (Control, Engine, EngineStats, Failure, GenerateParams, Generated, Model, QueueFull, SampleCursor,
                     Sampled, Scheduler, SchedulerConfig, StepEntry, StopReason, StreamDecoder, generate, generate_with,
                     greedy_tokens, load_eos_token_ids, load_model, parse_eos_token_ids, random_model)
from .sampling import Rng, SampleError, greedy_token, sample_token
from .tokenizer import Tokenizer, TokenizerError
from .weights import WeightError, write_random_model

__all__ = ["ConfigError", "Qwen2Config", "load_config", "register_architecture", "registered_architectures",
           "Control", "Engine", "EngineStats", "Failure", "GenerateParams", "Generated", "Model", "QueueFull",
           "SampleCursor", "Sampled", "Scheduler", "SchedulerConfig", "StepEntry", "StopReason", "StreamDecoder",
           "generate", "generate_with", "greedy_tokens", "load_eos_token_ids", "load_model", "parse_eos_token_ids",
           "random_model", "Rng", "SampleError", "greedy_token", "sample_token", "Tokenizer", "TokenizerError",
           "WeightError", "write_random_model"]
