"""Greedy and temperature sampling on the GPU.

Reference: ``Sampler`` (src/levanter/layers/sampler.py:15-81): logits in 32-bit; temperature 0
gives the argmax, otherwise a categorical draw from ``logits / temperature``; the log-probability
of the chosen token is ``scaled_logit - logsumexp(scaled_logits)``. The reference samples with
``fold_in(request key, position of the input token)`` (src/levanter/inference/jit_scheduler.py:141-156),
so a token's randomness depends on the request and the position only, not on the batch. Here the
draw is argmax(scaled logits + Gumbel noise) with noise from a counter-based generator keyed by
(request key, position, vocabulary entry). The reference has no top-k, top-p or penalties.
"""
from __future__ import annotations

from typing import Sequence, Tuple

import numpy as np
import torch

from levanter_amd.kernels.staging import pinned_pool

_MASK64 = (1 << 64) - 1


def _splitmix64(x: int) -> int:
    x = (x + 0x9E3779B97F4A7C15) & _MASK64
    z = x
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK64
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK64
    return z ^ (z >> 31)


def make_key(seed: int) -> Tuple[int, int]:
    """A 64-bit sampling key (two 32-bit words) from an integer seed (the reference's ``PRNGKey(seed)``)."""
    z = _splitmix64(int(seed) & _MASK64)
    return z & 0xFFFFFFFF, z >> 32


def fold_in(key: Tuple[int, int], data: int) -> Tuple[int, int]:
    """A new key from a key and an integer (the reference's ``jax.random.fold_in``; not the same bits)."""
    z = _splitmix64(((key[1] << 32) | key[0]) ^ _splitmix64(int(data) & _MASK64))
    return z & 0xFFFFFFFF, z >> 32


def _as_i32(word: int) -> int:
    return word - (1 << 32) if word >= (1 << 31) else word


class Sampler:
    def __init__(self, kernels, device):
        self.kernels = kernels
        self.device = torch.device(device)

    def __call__(self, logits: torch.Tensor, temperatures: Sequence[float], keys: Sequence[Tuple[int, int]],
                 positions: Sequence[int]) -> Tuple[torch.Tensor, torch.Tensor]:
        """logits float32 [R, V] on the device; one temperature, key and position per row.
        Returns (tokens int32 [R], log-probabilities float32 [R]) on the device."""
        r = logits.shape[0]
        assert len(temperatures) == len(keys) == len(positions) == r
        host = np.empty(4 * r, np.int32)
        host[:r] = np.asarray(temperatures, np.float32).view(np.int32)
        host[r:3 * r] = np.asarray([[_as_i32(k[0]), _as_i32(k[1])] for k in keys], np.int64).reshape(-1)
        host[3 * r:] = np.asarray(positions, np.int64)
        dev = torch.from_numpy(host) if self.device.type == "cpu" else pinned_pool().upload(host, self.device)
        out = torch.empty(2 * r, dtype=torch.int32, device=self.device)  # tokens, then log-probabilities: one copy back
        tokens, logprobs = out[:r], out[r:].view(torch.float32)
        self.kernels.sample(logits, dev[:r].view(torch.float32), dev[r:3 * r].view(r, 2), dev[3 * r:], tokens, logprobs)
        self._last_out = out
        return tokens, logprobs

    def to_host(self, logits: torch.Tensor, temperatures, keys, positions) -> Tuple[list, list]:
        """Sample and bring tokens and log-probabilities to the host with one copy (one synchronisation)."""
        return self.read(self.launch(logits, temperatures, keys, positions))

    def launch(self, logits: torch.Tensor, temperatures, keys, positions) -> "PendingSample":
        """Sample and start the copy of tokens and log-probabilities to the host without waiting for it. The tokens
        stay on the device too (``PendingSample.tokens``): the next step may be fed from there."""
        r = logits.shape[0]
        tokens, _ = self(logits, temperatures, keys, positions)
        out = self._last_out
        if self.device.type == "cpu":
            return PendingSample(r, tokens, out.clone(), None)
        host = pinned_pool().acquire(2 * r)
        host[:2 * r].copy_(out, non_blocking=True)
        done = torch.cuda.Event()
        done.record()
        return PendingSample(r, tokens, host, done)

    @staticmethod
    def read(pending: "PendingSample") -> Tuple[list, list]:
        if pending.done is not None:
            pending.done.synchronize()
        r = pending.rows
        result = pending.host[:r].tolist(), pending.host[r:2 * r].view(torch.float32).tolist()
        if pending.done is not None and pending.host is not None:
            pinned_pool().release(pending.host)  # a pinned buffer of the pool: the next sampling may take it
            pending.host = None
        return result


class PendingSample:
    """A sampling whose copy to the host is under way."""

    def __init__(self, rows: int, tokens: torch.Tensor, host: torch.Tensor, done):
        self.rows, self.tokens, self.host, self.done = rows, tokens, host, done
