"""A whole architecture defined outside the package: a configuration with config.json keys of its own, a spec
made of the toy parts, and its registration under a name of its own. Importing this module is all it takes;
a program started apart (bin/trace_run) learns of it through TNX_ARCHITECTURE_PACKAGES. A toy: it is no
model of anyone's.
"""
from dataclasses import dataclass
from typing import Any, ClassVar, Dict

import toy_parts
from transformers_neuronx_amd.config import register_architecture
from transformers_neuronx_amd.config.model_config import REQUIRED, ConfigError, ModelConfig


@dataclass(frozen=True)
class ToyTurnConfig(ModelConfig):
    architecture: ClassVar[str] = "ToyTurnLM"
    model_type: ClassVar[str] = "toy_turn"

    width: int = REQUIRED
    heads: int = REQUIRED
    shared_heads: int = REQUIRED      # key and value heads
    inner: int = REQUIRED
    words: int = REQUIRED             # the vocabulary
    longest: int = REQUIRED           # positions
    tiny: float = 1e-3                # the norms' eps
    turn_base: float = 100.0
    torch_dtype: str = "float32"

    def validate(self) -> None:
        if self.width % self.heads or (self.width // self.heads) % 16:
            raise ConfigError(f"key 'width' ({self.width}) must give 'heads' ({self.heads}) head sizes in 16s")
        if self.heads % self.shared_heads:
            raise ConfigError(f"key 'heads' ({self.heads}) must be a multiple of 'shared_heads' ({self.shared_heads})")

    def to_dict(self) -> Dict[str, Any]:
        d = super().to_dict()
        d["model_type"] = self.model_type
        return d


def toy_turn_spec(cfg: ToyTurnConfig):
    return toy_parts.toy_spec_rotating(width=cfg.width, heads=cfg.heads, kv_heads=cfg.shared_heads, inner=cfg.inner,
                                       vocab=cfg.words, positions=cfg.longest, eps=cfg.tiny, base=cfg.turn_base)


def plain_logits(cfg: ToyTurnConfig, weights, tokens):
    return toy_parts.toy_rotating_plain_logits(weights, tokens, width=cfg.width, heads=cfg.heads,
                                               kv_heads=cfg.shared_heads, eps=cfg.tiny, base=cfg.turn_base)


ARCHITECTURE = register_architecture("ToyTurnLM", "toy_turn", ToyTurnConfig, toy_turn_spec)

# two folders' worth of sizes that differ in every key
TOY_ONE = dict(width=96, heads=3, shared_heads=1, inner=72, words=157, longest=150, tiny=1e-3, turn_base=100.0)
TOY_TWO = dict(width=128, heads=4, shared_heads=2, inner=104, words=263, longest=200, tiny=1e-5, turn_base=33.0)
