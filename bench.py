#!/usr/bin/env python3
"""Benchmark: decode tokens per second of the GPT-2 7B shape on one MI355X, through the engine's own
scheduler, step function, cache and kernels.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 8] [--layers L] [--dtype bfloat16]

A step is one decode step of the whole batch. Prints ONE JSON line: the decode rate at the
default batch, the prefill rate of a 2,048-token prompt with its fraction of the MFMA peak, the
decode step's fraction of the HBM roofline, and the decode rates at batch 1 and 64.
Weights are random (N(0, 0.02), drawn on the GPU), token ids are seeded uniform-random: synthetic data.
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

# MI355X published peaks
HBM_BYTES_PER_S = 8.0e12
PEAK_FLOPS = {"bfloat16": 2.5e15, "float32": 157.3e12}


def load_baseline_config():
    """Layer sizes of BASELINE.json's configs[2] (the repo's gpt2_7b shape)."""
    return {"model_type": "gpt2", "n_layer": 32, "n_embd": 4096, "n_head": 32, "n_inner": 16384, "vocab_size": 50257,
            "n_positions": 2048, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--prompt-len", type=int, default=512)
    ap.add_argument("--layers", type=int, default=None, help="fewer layers than the configuration has (both numbers are reported)")
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--prefill-only", action="store_true", help="time the 2,048-token prefill alone (for profiling); prints its own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from levanter_amd.config import InferenceEngineConfig, LmConfig
    from levanter_amd.engine import InferenceEngine, Request

    raw = load_baseline_config()
    full_layers = raw["n_layer"]
    if args.layers is not None:
        raw["n_layer"] = args.layers
    cfg = LmConfig.from_dict(raw)
    ps = 16
    max_batch = max(args.batch, 1 if args.no_points else 64)
    ctx_end = args.prompt_len + args.warmup + args.steps + 1
    pages_per_seq = (max(ctx_end, 2048) + ps - 1) // ps
    ecfg = InferenceEngineConfig(max_pages=max_batch * ((ctx_end + ps - 1) // ps) + pages_per_seq, max_seqs=max_batch, page_size=ps,
                                 max_pages_per_seq=pages_per_seq, compute_dtype=args.dtype, max_prefill_size=2048,
                                 max_seqs_in_prefill=max_batch)
    t0 = time.time()
    engine = InferenceEngine.from_config(cfg, seed=0, config=ecfg)
    torch.cuda.synchronize()
    print(f"[bench] model ready in {time.time() - t0:.1f}s: {engine.model.weight_bytes() / 1e9:.2f} GB of weights", file=sys.stderr, flush=True)

    itemsize = 2 if args.dtype == "bfloat16" else 4
    L, D, F, V = cfg.n_layer, cfg.n_embd, cfg.inner_dim, cfg.vocab_size
    matrix_params = L * (3 * D * D + D * D + 2 * D * F)
    weight_bytes = (matrix_params + V * D) * itemsize + L * (3 * D + D + F + D + 4 * D) * 4 + 2 * D * 4
    kv_bytes_per_token = 2 * L * D * itemsize

    def prompts(batch, n, seed):
        g = torch.Generator().manual_seed(seed)
        return [torch.randint(0, V, (n,), generator=g).tolist() for _ in range(batch)]

    def decode_run(batch, steps, warmup, seed):
        """Prefill ``batch`` prompts, then time ``steps`` decode steps. Returns (seconds, mean context)."""
        engine.reset()
        reqs = [Request(prompt_tokens=p, request_id=i, max_new_tokens=warmup + steps + 8, temperature=0.0)
                for i, p in enumerate(prompts(batch, args.prompt_len, seed))]
        seqs = engine.enqueue_requests(reqs)
        while any(s.n_cached < s.prompt_len for s in seqs) or any(not s.generated for s in seqs):
            engine.step()
        for _ in range(warmup):
            engine.step()
        torch.cuda.synchronize()
        ctx0 = seqs[0].n_cached
        t = time.perf_counter()
        for _ in range(steps):
            engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert all(len(s.generated) >= warmup + steps for s in seqs), "the timed steps did not all decode the whole batch"
        ctx_mean = ctx0 + (steps + 1) / 2.0
        engine.reset()
        return dt, ctx_mean

    def prefill_run(T, reps):
        best = None
        for rep in range(reps):
            engine.reset()
            engine.enqueue_requests([Request(prompt_tokens=prompts(1, T, 50 + rep)[0], request_id=rep, max_new_tokens=1)])
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            d = time.perf_counter() - t
            best = d if best is None or d < best else best
        flops = 2.0 * T * matrix_params + 2.0 * T * T * D * L + 2.0 * D * V
        return {"value": round(T / best, 1), "tokens": T, "ms": round(best * 1e3, 3), "frac": round(flops / best / PEAK_FLOPS[args.dtype], 4)}

    if args.prefill_only:
        print(json.dumps({"prefill": prefill_run(2048, 4)}), flush=True)
        return 0

    dt, ctx_mean = decode_run(args.batch, args.steps, args.warmup, seed=1)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes + args.batch * ctx_mean * kv_bytes_per_token
    achieved = step_bytes / (dt / args.steps) / 1e9
    out = {
        "metric": "decode tok/s @ batch 8, GPT-2 7B shape, bf16" if args.batch == 8 else f"decode tok/s @ batch {args.batch}, GPT-2 7B shape",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": "gpt2_7b shape", "n_layer": L, "n_layer_full": full_layers, "n_embd": D, "n_head": cfg.n_head,
                   "head_dim": cfg.head_dim, "n_inner": F, "vocab_size": V, "n_positions": cfg.n_positions,
                   "global_batch": args.batch, "seq_len": args.prompt_len + args.steps, "prompt_len": args.prompt_len,
                   "page_size": ps, "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved / (HBM_BYTES_PER_S / 1e9), 4)},
    }
    if not args.no_points:
        # prefill of one 2,048-token prompt in one step (the logits of its last token)
        out["prefill"] = prefill_run(2048, 3)
        points = {}
        for b, steps in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            d, _ = decode_run(b, steps, min(args.warmup, 4), seed=2 + b)
            points[f"decode_b{b}"] = round(b * steps / d, 2)
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
