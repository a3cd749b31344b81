"""tokenizer_amd: a small inference engine for AMD MI355X (gfx950), built on hand-written HIP kernels."""
from . import models  # noqa: F401  (registers the architectures)
from .config import ConfigError, Qwen2Config, load_config, register_architecture, registered_architectures
from .engine import Engine, Model, StepEntry, load_model, random_model
from .weights import WeightError, write_random_model

__all__ = ["ConfigError", "Qwen2Config", "load_config", "register_architecture", "registered_architectures",
           "Engine", "Model", "StepEntry", "load_model", "random_model", "WeightError", "write_random_model"]
