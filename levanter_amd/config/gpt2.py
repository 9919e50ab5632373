"""Gpt2Config: the typed configuration of the GPT-2 architecture, under its config.json keys.

Reference: src/levanter/models/gpt2.py:34-129. The reference's field names (``seq_len``,
``hidden_dim``, ``num_layers``, ``num_heads``, ``upcast_attn``) map to the config.json keys
``n_positions``, ``n_embd``, ``n_layer``, ``n_head``, ``reorder_and_upcast_attn`` in
``from_hf_config`` (gpt2.py:102-117); this class keeps the config.json names. ``n_inner`` is
honoured (the reference fixes the feed-forward width at 4 * n_embd, gpt2.py:43,71).
"""
from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Any, Dict, Optional

from .lm_config import ConfigError, LmConfig

# src/levanter/utils/activation.py:18-40
ACTIVATION_NAMES = ("relu", "silu", "swish", "gelu", "gelu_new", "quick_gelu", "tanh")


@LmConfig.register_subclass("gpt2")
@dataclass(frozen=True)
class Gpt2Config(LmConfig):
    vocab_size: int = 50257
    n_positions: int = 1024
    n_embd: int = 768
    n_layer: int = 12
    n_head: int = 12
    n_inner: Optional[int] = None
    activation_function: str = "gelu_new"
    layer_norm_epsilon: float = 1e-5
    scale_attn_by_inverse_layer_idx: bool = False
    reorder_and_upcast_attn: bool = False
    initializer_range: float = 0.02
    tie_word_embeddings: bool = True
    use_bias: bool = True  # the reference's own flag (gpt2.py:57); absent from config.json means True
    scale_attn_weights: bool = True
    """A key of GPT-2's config.json that the reference does not read (gpt2.py:102-117): scores are always scaled by
    1/sqrt(head size) (src/levanter/layers/attention.py:153-154). ``false`` is refused rather than ignored."""
    attn_pdrop: float = 0.0
    embd_pdrop: float = 0.0
    resid_pdrop: float = 0.0

    def __post_init__(self):
        for name in ("vocab_size", "n_positions", "n_embd", "n_layer", "n_head"):
            v = getattr(self, name)
            if not isinstance(v, int) or isinstance(v, bool) or v <= 0:
                raise ConfigError(f"gpt2: {name} must be a positive integer, got {v!r}")
        if self.n_embd % self.n_head != 0:
            raise ConfigError(f"gpt2: n_embd={self.n_embd} is not divisible by n_head={self.n_head}")
        if self.n_inner is not None and (not isinstance(self.n_inner, int) or self.n_inner <= 0):
            raise ConfigError(f"gpt2: n_inner must be null or a positive integer, got {self.n_inner!r}")
        if self.activation_function not in ACTIVATION_NAMES:
            raise ConfigError(
                f"gpt2: unknown activation_function {self.activation_function!r}; known: {', '.join(ACTIVATION_NAMES)}"
            )
        if not self.layer_norm_epsilon > 0:
            raise ConfigError(f"gpt2: layer_norm_epsilon must be positive, got {self.layer_norm_epsilon!r}")
        if not self.scale_attn_weights:
            raise ConfigError("gpt2: scale_attn_weights=false is not supported (scores are always scaled by 1/sqrt(head size))")
        if not self.tie_word_embeddings:
            # the reference has no untied path: the head is the token table (gpt2.py:361-362)
            raise ConfigError("gpt2: tie_word_embeddings=false is not supported (the head is the token table)")

    # ---- derived sizes (gpt2.py:66-72) -----------------------------------------
    @property
    def head_dim(self) -> int:
        return self.n_embd // self.n_head

    @property
    def inner_dim(self) -> int:
        return self.n_inner if self.n_inner is not None else 4 * self.n_embd

    # ---- config.json ------------------------------------------------------------
    @classmethod
    def from_hf_config(cls, hf_config: Dict[str, Any]) -> "Gpt2Config":
        mt = hf_config.get("model_type", "gpt2")
        if mt != "gpt2":
            raise ConfigError(f"Gpt2Config cannot read a config.json of model_type {mt!r}")
        known = {f.name for f in fields(cls)}
        kwargs = {k: v for k, v in hf_config.items() if k in known}
        for required in ("vocab_size", "n_positions", "n_embd", "n_layer", "n_head"):
            if required not in kwargs:
                raise ConfigError(f"gpt2: config.json lacks the key {required!r}")
        try:
            return cls(**kwargs)
        except TypeError as e:  # wrong types that the dataclass cannot take
            raise ConfigError(f"gpt2: bad config.json: {e}") from None

    def to_hf_config(self) -> Dict[str, Any]:
        out = {"model_type": "gpt2", "architectures": ["GPT2LMHeadModel"]}
        for f in fields(self):
            out[f.name] = getattr(self, f.name)
        return out

    def model_spec(self):
        from levanter_amd.models.gpt2 import gpt2_model_spec

        return gpt2_model_spec(self)
