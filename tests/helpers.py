"""Helpers shared by the tests: building attention metadata and paged caches by hand."""
from __future__ import annotations

import os
import tempfile
from typing import Dict, List, Sequence, Tuple

import numpy as np
import torch

from levanter_amd.parts.base import AttentionMeta


def make_meta(runs: Sequence[Tuple[int, int]], device, tile_rows: int = 0) -> AttentionMeta:
    """runs: (q_len, kv_len after the step) per request. Tokens of a request are consecutive."""
    if tile_rows <= 0:
        tile_rows = 64
        if str(device) != "cpu":
            from levanter_amd.kernels import get_kernels

            tile_rows = get_kernels().prefill_tile_rows
    positions, token_seq, tile_list, decode = [], [], [], []
    t0 = 0
    for s, (q_len, kv_len) in enumerate(runs):
        start = kv_len - q_len
        positions += list(range(start, kv_len))
        token_seq += [s] * q_len
        if q_len == 1:
            decode.append(t0)
        else:
            for r0 in range(0, q_len, tile_rows):
                nr = min(tile_rows, q_len - r0)
                tile_list.append((start + r0 + nr, t0 + r0, nr))
        t0 += q_len
    tile_list.sort(key=lambda x: -x[0])  # falling key range, as the step function orders them
    tiles = [v for _, first, nr in tile_list for v in (first, nr)]

    def dev(x):
        return torch.tensor(x, dtype=torch.int32, device=device)

    return AttentionMeta(positions=dev(positions), token_seq=dev(token_seq),
                         prefill_tiles=dev(tiles).view(-1, 2) if tiles else None, n_prefill_tiles=len(tiles) // 2,
                         decode_tokens=dev(decode) if decode else None, n_decode=len(decode),
                         max_kv_len=max(k for _, k in runs))


def random_block_tables(kv_lens: Sequence[int], page_size: int, n_pages: int, seed: int, device):
    """Distinct shuffled pages for every request; unused entries are -1. Returns the table [S, B]."""
    rng = np.random.default_rng(seed)
    pages = rng.permutation(n_pages)
    nb = max((k + page_size - 1) // page_size for k in kv_lens)
    bt = np.full((len(kv_lens), nb), -1, np.int32)
    i = 0
    for s, k in enumerate(kv_lens):
        n = (k + page_size - 1) // page_size
        assert i + n <= n_pages, "not enough pages for the test"
        bt[s, :n] = pages[i:i + n]
        i += n
    return torch.tensor(bt, device=device)


def dest_for(bt: torch.Tensor, s: int, positions: Sequence[int], page_size: int) -> List[int]:
    return [int(bt[s, p // page_size]) * page_size + p % page_size for p in positions]


def write_model(raw_config: dict, seed: int, dtype=torch.float32) -> str:
    """A model folder with random weights in a fresh temporary directory."""
    from levanter_amd.config import LmConfig
    from levanter_amd.weights import write_random_model

    d = tempfile.mkdtemp(prefix="lev_model_")
    write_random_model(LmConfig.from_dict(raw_config), seed, d, dtype)
    return d


def read_weights(model_dir: str, dtype=torch.float64) -> Dict[str, torch.Tensor]:
    """The folder's tensors through the safetensors package (not the engine's reader)."""
    from safetensors.torch import load_file

    return {k: v.to(dtype) for k, v in load_file(os.path.join(model_dir, "model.safetensors")).items()}


def toy_rotary_unit() -> str:
    """The toy rotation's kernel (``toy_rotary.hip`` beside the tests) as a kernel unit of its own, registered with the
    build from outside the package; returns the unit's name."""
    import ctypes

    from levanter_amd.kernels import build

    if "toy_rotary" not in build.UNITS:
        P_, I_, L_, F_ = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float
        build.register_unit("toy_rotary", ["toy_rotary.hip"], source_dir=os.path.dirname(os.path.abspath(__file__)),
                            signatures={"toy_rotate": [P_, L_, P_, I_, I_, I_, F_, I_, P_]})
    return "toy_rotary"
