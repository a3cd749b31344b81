"""Configuration of the Qwen2 dense decoder, from its config.json keys.

Keys and checks follow qwen-infer/src/model.rs:25-42 and 714-738.  The window
keys are only needed when `use_sliding_window` is true; `head_dim`, if a file
names it, has to equal hidden_size / num_attention_heads (the reference derives
it, model.rs:739).
"""
from __future__ import annotations

import dataclasses

from .base import ConfigError, ModelConfig


@dataclasses.dataclass(frozen=True)
class Qwen2Config(ModelConfig):
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_hidden_layers: int
    num_attention_heads: int
    num_key_value_heads: int
    max_position_embeddings: int
    tie_word_embeddings: bool
    rope_theta: float
    rms_norm_eps: float
    hidden_act: str
    use_sliding_window: bool = False
    sliding_window: int | None = None
    max_window_layers: int | None = None
    head_dim: int | None = None

    def validate(self) -> None:
        if self.hidden_act != "silu":
            raise ConfigError(f"expected hidden_act silu, found {self.hidden_act}")
        for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                    "num_attention_heads", "num_key_value_heads", "max_position_embeddings"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"{key} must be positive, found {getattr(self, key)}")
        if self.hidden_size % self.num_attention_heads:
            raise ConfigError(f"hidden_size {self.hidden_size} does not divide into "
                              f"{self.num_attention_heads} heads")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"{self.num_attention_heads} query heads is not a multiple of "
                              f"{self.num_key_value_heads} kv heads")
        derived = self.hidden_size // self.num_attention_heads
        if self.head_dim is not None and self.head_dim != derived:
            raise ConfigError(f"head_dim {self.head_dim} differs from hidden_size / num_attention_heads "
                              f"= {derived}")
        if derived % 2:
            raise ConfigError(f"head size {derived} is odd; the rotation pairs the two halves of a head")
        if not self.rope_theta > 0:
            raise ConfigError(f"rope_theta must be positive, found {self.rope_theta}")
        if not self.rms_norm_eps >= 0:
            raise ConfigError(f"rms_norm_eps must not be negative, found {self.rms_norm_eps}")
        if self.use_sliding_window:
            if self.sliding_window is None or self.max_window_layers is None:
                raise ConfigError("use_sliding_window is true but sliding_window or max_window_layers is missing")
            if self.sliding_window < 0 or self.max_window_layers < 0:
                raise ConfigError("sliding_window and max_window_layers must not be negative")

    @property
    def derived_head_dim(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def window_for_layer(self, index: int) -> int | None:
        """`None` unless the flag is on and the layer is at or past max_window_layers (model.rs:909-915)."""
        if self.use_sliding_window and index >= self.max_window_layers:
            return self.sliding_window
        return None
