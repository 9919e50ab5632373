"""Requests and results, with the reference's names.

``Request`` (src/levanter/inference/engine.py:36-44), ``SeqDecodingParams``
(src/levanter/inference/jit_scheduler.py:44-63), ``GenerationResult`` (engine.py:636-640).
``max_num_tokens`` caps the total length, prompt included (jit_scheduler.py:101-105); the command
line's ``max_new_tokens`` is converted as the reference does (src/levanter/main/sample_lm.py:164).
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional, Sequence, Tuple, Union

INT32_MAX = 2**31 - 1


@dataclass
class SeqDecodingParams:
    max_num_tokens: int = INT32_MAX - 100000
    """Most tokens the sequence may reach, prompt included."""
    stop_tokens: Optional[Sequence[Sequence[int]]] = None
    """Stop sequences (lists of token ids); generation ends when the tokens so far end with one of them."""
    temperature: float = 0.0
    """0: greedy."""
    key: Union[None, int, Tuple[int, int]] = None
    """Sampling key of the request; None: derived from the engine's seed and the request id."""


@dataclass
class Request:
    prompt_tokens: List[int]
    request_id: int
    decode_params: Optional[SeqDecodingParams] = None
    n_generations: int = 1
    enable_logprobs: bool = False
    # shorthands used when decode_params is not given
    max_new_tokens: Optional[int] = None
    temperature: float = 0.0
    stop_tokens: Optional[Sequence[Sequence[int]]] = None
    key: Union[None, int, Tuple[int, int]] = None

    def __post_init__(self):
        self.prompt_tokens = [int(t) for t in self.prompt_tokens]
        if self.decode_params is None:
            total = INT32_MAX - 100000 if self.max_new_tokens is None else len(self.prompt_tokens) + int(self.max_new_tokens)
            self.decode_params = SeqDecodingParams(max_num_tokens=total, stop_tokens=self.stop_tokens,
                                                   temperature=float(self.temperature), key=self.key)


@dataclass
class GenerationResult:
    tokens: List[List[int]]
    """Generated tokens only (the prompt is not echoed), the stopping token included; ordered by request, then generation."""
    logprobs: Optional[List[List[float]]]
    total_generated: int
    finish_reasons: List[str] = field(default_factory=list)
    """"length", "stop", or "error: ..." per sequence."""
