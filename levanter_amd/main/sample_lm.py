"""Command line: sample from a model folder.

    python -m levanter_amd.main.sample_lm --config_path sample.yaml [--section.name value ...]
    python -m levanter_amd.main.sample_lm --hf_checkpoint DIR --prompt_ids "[[5, 17, 3]]" --max_new_tokens 16

Options carry the names and meanings of the reference's ``SampleLmConfig``
(src/levanter/main/sample_lm.py:31-61): ``hf_checkpoint`` (here: a local folder with config.json
and model.safetensors), ``tokenizer``, ``engine`` (``InferenceEngineConfig``), ``prompts``,
``stop_sequence``, ``max_new_tokens`` (192), ``temperature`` (0.7), ``seed`` (2), ``n_generations`` (1),
``n_rounds`` (4; the same batch is generated that many times, the first round includes set-up),
``profile`` (the reference starts its profiler from the second round on, sample_lm.py:137-152; here every round then prints
how its time divides into the host's own work, the launches among it, and waiting for the GPU). ``trainer.mp`` keeps the reference's precision string ("p=bfloat16,c=bfloat16"); its compute
part sets ``engine.compute_dtype``. Added: ``prompt_ids`` and ``stop_ids`` give token ids directly, so that
no tokenizer is needed; ``random_config`` / ``random_seed`` run a randomly initialised model of a
configuration instead of a checkpoint.
"""
from __future__ import annotations

import dataclasses
import json
import os
import sys
import time
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional, Union

from levanter_amd.config import ConfigError, InferenceEngineConfig, LmConfig
from levanter_amd.config.cli import parse_config


@dataclass
class TrainerConfig:
    """The part of the reference's trainer section that matters for sampling."""

    mp: Optional[str] = None  # e.g. "p=bfloat16,c=bfloat16" (src/levanter/config.py:39-51)
    seed: int = 0


@dataclass
class SampleLmConfig:
    checkpoint_path: Optional[str] = None
    hf_checkpoint: Optional[str] = None
    trainer: TrainerConfig = field(default_factory=TrainerConfig)
    model: Optional[Dict[str, Any]] = None
    tokenizer: Optional[str] = None
    engine: InferenceEngineConfig = field(default_factory=InferenceEngineConfig)
    prompts: Union[str, List[str], None] = None
    prompt_ids: Optional[List[List[int]]] = None
    stop_sequence: Optional[str] = "."
    stop_ids: Optional[List[int]] = None
    max_new_tokens: int = 192
    temperature: float = 0.7
    seed: int = 2
    n_generations: int = 1
    n_rounds: int = 4
    profile: bool = False
    random_config: Optional[str] = None
    random_seed: int = 0


def _compute_dtype(cfg: SampleLmConfig) -> str:
    mp = cfg.trainer.mp
    if not mp:
        return cfg.engine.compute_dtype
    parts = dict(p.split("=", 1) for p in mp.replace(" ", "").split(",") if "=" in p)
    names = {"bfloat16": "bfloat16", "bf16": "bfloat16", "float32": "float32", "f32": "float32", "fp32": "float32"}
    c = parts.get("c", parts.get("compute", cfg.engine.compute_dtype))
    if c not in names:
        raise ConfigError(f"trainer.mp: compute dtype {c!r} is not supported (bfloat16 or float32)")
    return names[c]


def _load_tokenizer(path: Optional[str], model_dir: Optional[str]):
    for cand in (path, model_dir):
        if not cand:
            continue
        f = cand if os.path.isfile(cand) else os.path.join(cand, "tokenizer.json")
        if os.path.isfile(f):
            from tokenizers import Tokenizer

            return Tokenizer.from_file(f)
    return None


def main(config: SampleLmConfig) -> int:
    if config.checkpoint_path is not None:
        raise ConfigError("checkpoint_path (a training checkpoint of the reference) is not supported; give hf_checkpoint, a folder with "
                          "config.json and model.safetensors")
    if (config.hf_checkpoint is None) == (config.random_config is None):
        raise ConfigError("give exactly one of hf_checkpoint (a model folder) and random_config (a config.json for random weights)")

    from levanter_amd.engine import InferenceEngine, Request, SeqDecodingParams
    from levanter_amd.sampling import fold_in, make_key

    ecfg = dataclasses.replace(config.engine, compute_dtype=_compute_dtype(config))
    t0 = time.time()
    if config.hf_checkpoint is not None:
        engine = InferenceEngine.from_pretrained(config.hf_checkpoint, ecfg)
    else:
        with open(config.random_config) as f:
            engine = InferenceEngine.from_config(LmConfig.from_dict(json.load(f)), config.random_seed, ecfg)
    print(f"model loaded in {time.time() - t0:.2f} s ({ecfg.compute_dtype})", flush=True)

    tokenizer = _load_tokenizer(config.tokenizer, config.hf_checkpoint)
    if config.prompt_ids is not None:
        prompt_ids = [[int(t) for t in p] for p in config.prompt_ids]
    else:
        if config.prompts is None:
            raise ConfigError("give prompts (needs a tokenizer.json) or prompt_ids")
        if tokenizer is None:
            raise ConfigError("prompts are text but no tokenizer.json was found (tokenizer: a file or folder); or give prompt_ids")
        prompts = [config.prompts] if isinstance(config.prompts, str) else list(config.prompts)
        prompt_ids = [tokenizer.encode(p, add_special_tokens=False).ids for p in prompts]

    stop = None
    if config.stop_ids is not None:
        stop = [[int(t) for t in config.stop_ids]]
    elif config.stop_sequence is not None and tokenizer is not None:
        ids = tokenizer.encode(config.stop_sequence, add_special_tokens=False).ids
        if len(ids) == 0:
            raise ConfigError("Stop sequence must be non-empty")
        stop = [ids]

    base_key = make_key(ecfg.seed)
    for r in range(config.n_rounds):
        if r == 0:
            for i, toks in enumerate(prompt_ids):
                print(f"prompt {i} ({len(toks)} tokens): {toks}")
        time_in = time.time()
        reqs = [Request(prompt_tokens=toks, request_id=ridx,
                        decode_params=SeqDecodingParams(max_num_tokens=len(toks) + config.max_new_tokens, stop_tokens=stop,
                                                        temperature=config.temperature, key=fold_in(base_key, ridx)),
                        n_generations=config.n_generations)
                for ridx, toks in enumerate(prompt_ids)]
        before = dict(engine.stats)
        result = engine.generate(reqs)
        dt = time.time() - time_in
        print(f"round {r}: {result.total_generated} tokens in {len(result.tokens)} sequences, {dt:.2f} s "
              f"({result.total_generated / max(dt, 1e-9):.1f} tok/s)", flush=True)
        if config.profile:
            d = {k: engine.stats[k] - before[k] for k in before}
            n = max(1, d["commits"])
            print(f"round {r} profile: {d['steps']} steps of {d['tokens_in']} tokens in all; a step took the host {1e3 * (d['step_s'] - d['wait_s']) / n:.3f} ms "
                  f"({1e3 * d['launch_s'] / n:.3f} ms of it planning tables and launching kernels) and {1e3 * d['wait_s'] / n:.3f} ms of waiting for the GPU",
                  flush=True)
        for seq_id, out in enumerate(result.tokens):
            print(f"round {r} sequence {seq_id} ({len(out)} tokens, {result.finish_reasons[seq_id]}): {out}")
            if tokenizer is not None:
                print(f"round {r} sequence {seq_id} text: {tokenizer.decode(out, skip_special_tokens=True)}")
    return 0


if __name__ == "__main__":
    try:
        sys.exit(main(parse_config(SampleLmConfig)))
    except ConfigError as e:
        print(f"error: {e}", file=sys.stderr)
        sys.exit(2)
