"""From a model folder (or a configuration and a seed) to a runnable model and its runner.

The model class is chosen by ``config.json`` through the registry, as the reference does with
``config.model_type`` and ``converter.load_pretrained`` (src/levanter/main/sample_lm.py:64-89,
src/levanter/compat/hf_checkpoints.py:609-701)."""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from levanter_amd.cache import CacheManager, group_units, pages_per_group
from levanter_amd.config import InferenceEngineConfig, LmConfig
from levanter_amd.kernels import get_kernels
from levanter_amd.parts import BuildEnv, DecoderLm
from levanter_amd.weights import load_tensors, random_tensors

DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32}


def resolve_dtype(dtype) -> torch.dtype:
    if isinstance(dtype, torch.dtype):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype}")
        return dtype
    try:
        return DTYPES[str(dtype)]
    except KeyError:
        raise ValueError(f"compute dtype must be bfloat16 or float32, got {dtype!r}") from None


def make_env(dtype, device: Optional[str] = None) -> BuildEnv:
    """The build environment on the GPU; raises if there is none (no CPU path)."""
    kernels = get_kernels()
    dev = torch.device(device or "cuda:0")
    return BuildEnv(dtype=resolve_dtype(dtype), device=dev, kernels=kernels)


def load_model(model_dir: str, env: BuildEnv) -> Tuple[LmConfig, DecoderLm]:
    config = LmConfig.load(model_dir)
    spec = config.model_spec()
    tensors = load_tensors(model_dir, spec, device="cpu")
    return config, DecoderLm(spec, tensors, env)


def random_model(config: LmConfig, seed: int, env: BuildEnv) -> DecoderLm:
    """A model with random weights drawn on the model's device (no folder is written)."""
    spec = config.model_spec()
    tensors = random_tensors(spec, seed, dtype=env.dtype, device=env.device)
    return DecoderLm(spec, tensors, env)


def _free_device_bytes(device) -> int:
    free, _total = torch.cuda.mem_get_info(device)
    return int(free)


def make_cache(model: DecoderLm, cfg: InferenceEngineConfig, env: Optional[BuildEnv] = None, free_bytes=None) -> CacheManager:
    """The cache manager of a model under an engine configuration. Every cache group gets a pool of its own size:
    ``max_pages`` (or ``max_seqs * max_pages_per_seq``) pages where all keys are kept, what the window and a step's
    longest portion can touch where only a window is; with ``max_pages="auto"`` what is free on the device now (call
    this once the weights are there) less ``cache_memory_reserve_gib``. ``free_bytes``: a stand-in for the query."""
    requirements = model.cache_requirements()
    by_req, _ = group_units(requirements)
    if free_bytes is None and env is not None and env.device.type == "cuda":
        free_bytes = lambda: _free_device_bytes(env.device)
    itemsize = 4 if cfg.compute_dtype == "float32" else 2
    counts = pages_per_group([(req, len(units)) for req, units in by_req.items()], max_pages=cfg.max_pages, page_size=cfg.page_size,
                             max_seqs=cfg.max_seqs, max_pages_per_seq=cfg.max_pages_per_seq,
                             longest_portion=cfg.imputed_max_prefill_size, itemsize=itemsize, free_bytes=free_bytes,
                             reserve_bytes=int(cfg.cache_memory_reserve_gib * (1 << 30)))
    return CacheManager(requirements, n_pages=counts, page_size=cfg.page_size, max_seqs=cfg.max_seqs,
                        max_pages_per_seq=cfg.max_pages_per_seq)
