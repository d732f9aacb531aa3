"""OPT's configuration: the keys of its config.json (reference: opt/config.py:22-40)."""
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional, Tuple

from ..config.model_config import REQUIRED, ConfigError, ModelConfig

ACTIVATIONS: Tuple[str, ...] = ("relu", "gelu", "gelu_new")


@dataclass(frozen=True)
class OPTConfig(ModelConfig):
    """The keys of an OPT config.json.

    The reference copies ten of them (opt/config.py:22-40: activation_function,
    eos/pad_token_id, ffn_dim, hidden_size, max_position_embeddings,
    num_attention_heads, num_hidden_layers, vocab_size, word_embed_proj_dim) and
    refuses `do_layer_norm_before=false` (:23-24); the full key set is that of
    opt/gen_random_pretrained.py:105-140. Here every option of the family is
    honoured: post-norm order, embedding width different from the hidden width,
    no biases, norms without affine parameters.
    `layer_norm_eps` is not a key of published OPT checkpoints; it defaults to the
    value the reference fixes in code (hlo.py:51, 1e-5).
    """

    architecture: ClassVar[str] = "OPTForCausalLM"
    model_type: ClassVar[str] = "opt"

    vocab_size: int = REQUIRED
    hidden_size: int = REQUIRED
    num_hidden_layers: int = REQUIRED
    num_attention_heads: int = REQUIRED
    ffn_dim: int = REQUIRED
    max_position_embeddings: int = REQUIRED
    word_embed_proj_dim: Optional[int] = None
    do_layer_norm_before: bool = True
    activation_function: str = "relu"
    enable_bias: bool = True
    layer_norm_elementwise_affine: bool = True
    layer_norm_eps: float = 1e-5
    tie_word_embeddings: bool = True
    # pre-norm models only: true drops the norm before the head (a key of published OPT config.json files,
    # opt/gen_random_pretrained.py:114; the reference never reads it and always applies the norm)
    _remove_final_layer_norm: bool = False
    bos_token_id: int = 2
    eos_token_id: int = 2
    pad_token_id: int = 1
    init_std: float = 0.02
    torch_dtype: str = "float16"

    def __post_init__(self):
        if self.word_embed_proj_dim is None:
            object.__setattr__(self, "word_embed_proj_dim", self.hidden_size)

    @staticmethod
    def _coerce(f, value):
        if f.name == "word_embed_proj_dim":
            if isinstance(value, bool) or not isinstance(value, int):
                raise ConfigError(f"key 'word_embed_proj_dim' must be an integer, got {value!r}")
            return value
        return ModelConfig._coerce(f, value)

    @property
    def head_size(self) -> int:
        return self.hidden_size // self.num_attention_heads

    def validate(self) -> None:
        for key in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                    "ffn_dim", "max_position_embeddings", "word_embed_proj_dim"):
            if getattr(self, key) <= 0:
                raise ConfigError(f"key '{key}' must be positive, got {getattr(self, key)}")
        if self.hidden_size % self.num_attention_heads:
            raise ConfigError(
                f"key 'hidden_size' ({self.hidden_size}) must be a multiple of "
                f"'num_attention_heads' ({self.num_attention_heads})")
        if self.activation_function not in ACTIVATIONS:
            raise ConfigError(
                f"key 'activation_function' must be one of {ACTIVATIONS}, got {self.activation_function!r}")
        if self.layer_norm_eps <= 0:
            raise ConfigError(f"key 'layer_norm_eps' must be positive, got {self.layer_norm_eps}")
        if self.torch_dtype not in ("float32", "float16", "bfloat16"):
            raise ConfigError(f"key 'torch_dtype' must be float32, float16 or bfloat16, got {self.torch_dtype!r}")

    def to_dict(self) -> Dict[str, Any]:
        d = super().to_dict()
        d["model_type"] = self.model_type
        return d
