"""Tiny Qwen2 configurations for the tests.  They differ in every size and option."""
import numpy as np

_BASE = {"architectures": ["Qwen2ForCausalLM"], "hidden_act": "silu", "model_type": "qwen2"}

TINY = {
    # name: (config.json keys, weight seed)
    "A": ({**_BASE, "num_hidden_layers": 2, "hidden_size": 64, "num_attention_heads": 4, "num_key_value_heads": 2,
           "intermediate_size": 128, "vocab_size": 256, "rope_theta": 10000.0, "rms_norm_eps": 1e-6,
           "tie_word_embeddings": True, "max_position_embeddings": 128, "use_sliding_window": False,
           "sliding_window": 128, "max_window_layers": 2}, 0),
    "B": ({**_BASE, "num_hidden_layers": 3, "hidden_size": 96, "num_attention_heads": 3, "num_key_value_heads": 1,
           "intermediate_size": 272, "vocab_size": 384, "rope_theta": 1000000.0, "rms_norm_eps": 1e-5,
           "tie_word_embeddings": False, "max_position_embeddings": 256, "use_sliding_window": False,
           "sliding_window": 256, "max_window_layers": 3}, 2),
    # A window on the upper layers only: two cache groups, pages given back behind the window.
    "C": ({**_BASE, "num_hidden_layers": 4, "hidden_size": 80, "num_attention_heads": 5, "num_key_value_heads": 5,
           "intermediate_size": 176, "vocab_size": 320, "rope_theta": 500000.0, "rms_norm_eps": 3e-6,
           "tie_word_embeddings": True, "max_position_embeddings": 512, "use_sliding_window": True,
           "sliding_window": 21, "max_window_layers": 1}, 5),
}


def random_ids(vocab: int, length: int, seed: int) -> list[int]:
    return [int(v) for v in np.random.default_rng(seed).integers(0, vocab, size=length)]
