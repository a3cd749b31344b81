"""A toy model frame defined outside the package: the Qwen2 parts behind an embedding that is multiplied by a
constant of its own config.json key, with a cap on the logits.  Importing this module registers the frame and an
architecture that uses it; programs started by name import it through TOKENIZER_AMD_PLUGINS.  It is a test's toy, not
a model of anyone's."""
import dataclasses

import torch

from tokenizer_amd.config import Qwen2Config, register_architecture, registered_architectures
from tokenizer_amd.models.qwen2 import qwen2_spec
from tokenizer_amd.parts import FRAMES, DecoderModel

ARCHITECTURE = "ToyScaledFrameForCausalLM"


@dataclasses.dataclass(frozen=True)
class ToyScaledConfig(Qwen2Config):
    embedding_scale: float = 1.0
    logit_cap: float = 0.0            # 0: none; else logits = cap * tanh(logits / cap)


if "toy_scaled_decoder" not in FRAMES.kinds():
    @FRAMES.register("toy_scaled_decoder")
    class ToyScaledDecoder(DecoderModel):
        def embed(self, ctx):
            return super().embed(ctx).mul_(float(self.spec.options["embedding_scale"]))

        def logits(self, residual, delta, ctx):
            out = super().logits(residual, delta, ctx)
            cap = float(self.spec.options["logit_cap"])
            return out if cap == 0.0 else torch.tanh(out / cap) * cap


def toy_scaled_spec(cfg: ToyScaledConfig):
    return dataclasses.replace(qwen2_spec(cfg), architecture=ARCHITECTURE, frame="toy_scaled_decoder",
                               options={"embedding_scale": cfg.embedding_scale, "logit_cap": cfg.logit_cap})


if ARCHITECTURE not in registered_architectures():
    register_architecture(ARCHITECTURE, ToyScaledConfig, toy_scaled_spec)
