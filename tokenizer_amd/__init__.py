"""tokenizer_amd: a small inference engine for AMD MI355X (gfx950), built on hand-written HIP kernels.

The names follow the library of the reference's `qwen-infer` crate (qwen-infer/src/lib.rs:14-24):
`load_model`, `generate`, `generate_with`, `greedy_tokens`, `GenerateParams`, `Generated`, `StopReason`,
`Control`, `SampleCursor`, `greedy_token`, `sample_token`, `StreamDecoder`, `parse_eos_token_ids`,
`load_eos_token_ids`, and `Tokenizer.load_qwen`; beside them the engine's own `Engine` (one `step()` over a
mixed batch), `Scheduler`, `random_model`, `write_random_model` and `load_tokenizer` (the tokenizer of the kind a
folder's tokenizer.json declares).

Parts, frames, architectures and tokenizer kinds are registered by importing the module that defines them.  For
programs that are started by name (`bin/trace_run`, `bin/qwen-infer`, `bench.py`), the environment variable
`TOKENIZER_AMD_PLUGINS` lists modules (comma-separated, importable from `sys.path`) that are imported once the
package is set up, so a user's own architecture reaches them without a change to the package.
"""
from . import models  # noqa: F401  (registers the architectures)
from .config import ConfigError, Qwen2Config, load_config, register_architecture, registered_architectures
from .engine import (Control, Engine, EngineStats, Failure, GenerateParams, Generated, Model, QueueFull, SampleCursor,
                     Sampled, Scheduler, SchedulerConfig, StepEntry, StopReason, StreamDecoder, generate, generate_with,
                     greedy_tokens, load_eos_token_ids, load_model, parse_eos_token_ids, random_model)
from .sampling import Rng, SampleError, greedy_token, sample_token
from .tokenizer import Tokenizer, TokenizerError, load_tokenizer, register_tokenizer
from .weights import WeightError, write_random_model

__all__ = ["ConfigError", "Qwen2Config", "load_config", "register_architecture", "registered_architectures",
           "Control", "Engine", "EngineStats", "Failure", "GenerateParams", "Generated", "Model", "QueueFull",
           "SampleCursor", "Sampled", "Scheduler", "SchedulerConfig", "StepEntry", "StopReason", "StreamDecoder",
           "generate", "generate_with", "greedy_tokens", "load_eos_token_ids", "load_model", "parse_eos_token_ids",
           "random_model", "Rng", "SampleError", "greedy_token", "sample_token", "Tokenizer", "TokenizerError",
           "WeightError", "write_random_model", "load_tokenizer", "register_tokenizer"]


def _import_plugins() -> None:
    import importlib
    import os
    for name in filter(None, (part.strip() for part in os.environ.get("TOKENIZER_AMD_PLUGINS", "").split(","))):
        importlib.import_module(name)


_import_plugins()
