"""InferenceEngineConfig: memory and scheduling options of the engine.

Names and meanings follow the reference's ``InferenceEngineConfig``
(src/levanter/inference/engine.py:60-111) wherever the option still means something on one
GPU with a host-side scheduler; the differences are stated per field.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Union

from .lm_config import ConfigError


@dataclass(frozen=True)
class InferenceEngineConfig:
    max_pages: Union[None, int, str] = None
    """Pages in the pool of each cache group that keeps all keys (a group that keeps a window takes what it can use).
    None: ``max_seqs * max_pages_per_seq`` (engine.py:108-111). "auto": what is free on the GPU once the weights are
    loaded, less ``cache_memory_reserve_gib``, and at most ``max_seqs * max_pages_per_seq``. (Ours.)"""
    cache_memory_reserve_gib: float = 8.0
    """With ``max_pages="auto"``: device memory left alone for activations and kernel workspaces. (Ours.)"""
    max_seqs: int = 16
    """Most requests that are live (hold a slot) at a time (engine.py:66)."""
    page_size: int = 16
    """Tokens per page; a multiple of 16. (The reference's default is 128, engine.py:68.)"""
    max_pages_per_seq: int = 64
    """Most pages one request may hold: its length is at most page_size * max_pages_per_seq (engine.py:70)."""
    compute_dtype: str = "bfloat16"
    """Dtype of weights, activations and the cache: "bfloat16" or "float32" (engine.py:72)."""
    max_queued_tokens: int = 512
    """Kept for compatibility (engine.py:74): the reference's device-side token queue has no
    counterpart here, decoded tokens wait on the host."""
    max_seqs_in_prefill: int = 16
    """Most requests that contribute a portion of their prompt to one step (engine.py:76)."""
    max_prefill_size: Optional[int] = None
    """Most prompt tokens in one step (engine.py:80). Longer prompts are cut into portions
    (the reference can never admit them). None: page_size * max_pages_per_seq, capped at 2048."""
    max_tokens_per_round: Optional[int] = None
    """Most decoded tokens in one step; None: max_seqs (engine.py:88)."""
    max_rounds: int = 8
    """Decode steps run back to back before the queue is looked at again for admission (engine.py:90)."""
    max_stop_seqs: int = 4
    """Most stop sequences per request (engine.py:94)."""
    max_stop_tokens: int = 16
    """Most tokens in one stop sequence (engine.py:96)."""
    seed: int = 0
    """Seed from which per-request sampling keys are derived (engine.py:100)."""
    enable_logprobs: bool = False
    """Return the log-probability of every generated token (engine.py:102)."""
    decode_lookahead: bool = True
    """Launch the next step of single tokens before the tokens of the running one are read back. (Ours.)"""

    def __post_init__(self):
        if self.page_size <= 0 or self.page_size % 16 != 0:
            raise ConfigError(f"page_size must be a positive multiple of 16, got {self.page_size}")
        if self.compute_dtype not in ("bfloat16", "float32"):
            raise ConfigError(f"compute_dtype must be 'bfloat16' or 'float32', got {self.compute_dtype!r}")
        for name in ("max_seqs", "max_pages_per_seq", "max_seqs_in_prefill", "max_rounds"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{name} must be positive, got {getattr(self, name)}")
        if isinstance(self.max_pages, str):
            if self.max_pages != "auto":
                raise ConfigError(f'max_pages must be a positive number, null or "auto", got {self.max_pages!r}')
        elif self.max_pages is not None and self.max_pages <= 0:
            raise ConfigError(f"max_pages must be positive, got {self.max_pages}")
        if self.cache_memory_reserve_gib < 0:
            raise ConfigError(f"cache_memory_reserve_gib must not be negative, got {self.cache_memory_reserve_gib}")

    @property
    def imputed_max_pages(self) -> int:
        """The page count of a group that keeps all keys, where it is known without asking the device."""
        if self.max_pages == "auto":
            raise ConfigError('max_pages="auto" is resolved when the cache is made, from the free device memory')
        return int(self.max_pages) if self.max_pages is not None else int(self.max_seqs * self.max_pages_per_seq)

    @property
    def max_len_per_seq(self) -> int:
        return self.page_size * self.max_pages_per_seq

    @property
    def imputed_max_prefill_size(self) -> int:
        if self.max_prefill_size is not None:
            return int(self.max_prefill_size)
        return min(self.max_len_per_seq, 2048)

    @property
    def imputed_max_tokens_per_round(self) -> int:
        return int(self.max_tokens_per_round) if self.max_tokens_per_round is not None else self.max_seqs
