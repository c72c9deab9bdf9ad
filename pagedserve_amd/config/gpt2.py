"""Typed GPT-2 configuration, read from the keys that a GPT-2 ``config.json`` holds.

The reference fills an engine-neutral dataclass from a Hugging Face config object
(src/model/gpt2.py:32-44, fields at src/model/paged_decoder.py:29-41) and rejects
what it cannot run (src/model/gpt2.py:23-30).  Here the JSON file itself is the
source, and no size or constant that it gives is repeated in code.
"""

from dataclasses import dataclass
from typing import Optional

from .base import ConfigError, require_int as _require_int

_TANH_GELU = ("gelu_new", "gelu_pytorch_tanh")
_ERF_GELU = ("gelu",)


@dataclass(frozen=True)
class GPT2Config:
    """The options of ``GPT2LMHeadModel`` that change what is computed."""

    n_layer: int
    n_embd: int
    n_head: int
    n_inner: int
    n_positions: int
    vocab_size: int
    layer_norm_epsilon: float
    activation_function: str
    scale_attn_by_inverse_layer_idx: bool
    tie_word_embeddings: bool
    eos_token_id: Optional[int]

    architecture = "GPT2LMHeadModel"

    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @property
    def activation_kind(self) -> str:
        """``"gelu_tanh"`` or ``"gelu_erf"``: the two forms of
        src/model/paged_decoder.py:273-280."""
        return "gelu_tanh" if self.activation_function in _TANH_GELU else "gelu_erf"

    @classmethod
    def from_dict(cls, raw) -> "GPT2Config":
        n_embd = _require_int(raw, "n_embd")
        n_head = _require_int(raw, "n_head")
        if n_embd % n_head != 0:
            # src/model/gpt2.py:23-24
            raise ConfigError(f"n_embd ({n_embd}) must be divisible by n_head ({n_head})")
        if raw.get("add_cross_attention", False):
            # src/model/gpt2.py:25-26
            raise ConfigError("GPT-2 with cross-attention is not supported")
        if raw.get("scale_attn_weights", True) is False:
            raise ConfigError("scale_attn_weights=false is not supported")
        if raw.get("reorder_and_upcast_attn", False):
            # only changes the precision of the score product; scores here are 32-bit anyway
            pass
        activation = raw.get("activation_function", "gelu_new")
        if activation not in _TANH_GELU + _ERF_GELU:
            raise ConfigError(
                f"activation_function {activation!r} is not supported; "
                f"known: {', '.join(_TANH_GELU + _ERF_GELU)}")
        n_inner = raw.get("n_inner")
        if n_inner is None:
            n_inner = 4 * n_embd  # src/model/gpt2.py:38
        elif isinstance(n_inner, bool) or not isinstance(n_inner, int) or n_inner < 1:
            raise ConfigError(f"config.json 'n_inner' must be a positive integer or null, got {n_inner!r}")
        # The reference reads the alias max_position_embeddings (src/model/gpt2.py:39).
        if "n_positions" in raw:
            n_positions = _require_int(raw, "n_positions")
        else:
            n_positions = _require_int(raw, "max_position_embeddings")
        eps = raw.get("layer_norm_epsilon", 1e-5)
        if not isinstance(eps, (int, float)) or isinstance(eps, bool) or not eps > 0:
            raise ConfigError(f"layer_norm_epsilon must be a positive number, got {eps!r}")
        eos = raw.get("eos_token_id")
        if eos is not None and (isinstance(eos, bool) or not isinstance(eos, int)):
            raise ConfigError(f"eos_token_id must be an integer or null, got {eos!r}")
        return cls(
            n_layer=_require_int(raw, "n_layer"),
            n_embd=n_embd,
            n_head=n_head,
            n_inner=n_inner,
            n_positions=n_positions,
            vocab_size=_require_int(raw, "vocab_size"),
            layer_norm_epsilon=float(eps),
            activation_function=activation,
            scale_attn_by_inverse_layer_idx=bool(raw.get("scale_attn_by_inverse_layer_idx", False)),
            tie_word_embeddings=bool(raw.get("tie_word_embeddings", True)),
            eos_token_id=eos,
        )

    def to_dict(self) -> dict:
        """The config.json that reads back as this configuration."""
        return {
            "architectures": [self.architecture],
            "model_type": "gpt2",
            "n_layer": self.n_layer,
            "n_embd": self.n_embd,
            "n_head": self.n_head,
            "n_inner": self.n_inner,
            "n_positions": self.n_positions,
            "vocab_size": self.vocab_size,
            "layer_norm_epsilon": self.layer_norm_epsilon,
            "activation_function": self.activation_function,
            "scale_attn_by_inverse_layer_idx": self.scale_attn_by_inverse_layer_idx,
            "tie_word_embeddings": self.tie_word_embeddings,
            "eos_token_id": self.eos_token_id,
        }
