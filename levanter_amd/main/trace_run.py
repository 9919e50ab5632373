"""The program behind ``bin/trace_run``: replays a trace of steps through ``ModelRunner.step``."""
from __future__ import annotations

import argparse
import json
import os
import sys
from typing import Dict



def main(argv=None) -> int:
    ap = argparse.ArgumentParser(prog="trace_run", description="feed token ids through a model step by step, write logits")
    ap.add_argument("--model", help="folder with config.json and model.safetensors")
    ap.add_argument("--random-config", help="instead of --model: a config.json (a file, or the JSON itself) whose model gets random weights "
                                            "drawn from --seed, the same as a folder written from that configuration and seed holds")
    ap.add_argument("--seed", type=int, default=0, help="with --random-config: the seed of the weights")
    ap.add_argument("--dtype", required=True, choices=["bfloat16", "float32"])
    ap.add_argument("--out", required=True, help="folder for <step>.f32 files")
    ap.add_argument("--max-tokens", type=int, required=True,
                    help="most tokens live requests hold at any time (each rounded up to a multiple of 64)")
    ap.add_argument("--page-size", type=int, default=16)
    ap.add_argument("--max-seqs", type=int, default=8)
    args = ap.parse_args(argv)
    if (args.model is None) == (args.random_config is None):
        ap.error("give either --model or --random-config")

    print("trace_run: loading torch and the HIP library ...", file=sys.stderr, flush=True)
    import torch  # noqa: F401

    from levanter_amd.cache import SequenceHandle
    from levanter_amd.config import InferenceEngineConfig
    from levanter_amd.engine import ModelRunner, StepEntry
    from levanter_amd.engine.loading import load_model, make_cache, make_env

    env = make_env(args.dtype)
    if args.model is not None:
        config, model = load_model(args.model, env)
    else:
        from levanter_amd.config import LmConfig
        from levanter_amd.parts import DecoderLm
        from levanter_amd.weights import random_tensors

        raw = args.random_config
        if not raw.lstrip().startswith("{"):
            with open(raw, encoding="utf-8") as f:
                raw = f.read()
        config = LmConfig.from_dict(json.loads(raw))
        spec = config.model_spec()
        # drawn on the CPU, stored in the compute dtype: tensor for tensor what write_random_model puts into a folder
        model = DecoderLm(spec, random_tensors(spec, args.seed, dtype=env.dtype, device="cpu"), env)
    ps = args.page_size
    n_pages = max(1, (args.max_tokens + ps - 1) // ps)
    if 64 % ps != 0 and ps % 64 != 0:  # counts are rounded to 64, pages are not: every live request may need one page more
        n_pages += args.max_seqs
    longest = args.max_tokens if model.max_positions is None else min(args.max_tokens, model.max_positions)
    ecfg = InferenceEngineConfig(max_pages=n_pages, max_seqs=args.max_seqs, page_size=ps,
                                 max_pages_per_seq=max(1, (longest + ps - 1) // ps), compute_dtype=args.dtype)
    cache = make_cache(model, ecfg)
    runner = ModelRunner(model, cache, env)
    os.makedirs(args.out, exist_ok=True)
    print(f"trace_run: ready ({config.model_type_name}, {args.dtype}, {n_pages} pages of {ps})", file=sys.stderr, flush=True)

    live: Dict[str, SequenceHandle] = {}
    for line in sys.stdin:
        line = line.strip()
        if not line:
            continue
        rec = json.loads(line)
        step = rec["step"]
        entries = []
        for e in rec.get("entries", []):
            rid = str(e["id"])
            if rid not in live:
                live[rid] = cache.open(rid)
            entries.append(StepEntry(live[rid], [int(t) for t in e["tokens"]], [int(w) for w in e.get("want", [])]))
        logits = runner.step(entries)
        if logits.shape[0] > 0:
            arr = logits.detach().to("cpu", torch.float32).contiguous().numpy().astype("<f4", copy=False)
            arr.tofile(os.path.join(args.out, f"{step}.f32"))
        else:
            torch.cuda.synchronize()
        for rid in rec.get("end", []):
            h = live.pop(str(rid), None)
            if h is not None:
                cache.close(h)
        print(f"done {step}", flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
