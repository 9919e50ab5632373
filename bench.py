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


GENERATED = 256  # the benchmark's requests generate this many tokens after their prompt


def load_baseline_config():
    """Layer sizes of the reference's gpt2_7b configuration (config/gpt2_7b.yaml) with GPT-2's vocabulary."""
    return {"model_type": "gpt2", "n_layer": 32, "n_embd": 4096, "n_head": 32, "n_inner": 16384, "vocab_size": 50257,
            "n_positions": 2048, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}


# the other sizes of the reference's configurations (config/gpt2_xl.yaml, config/gpt2_20b.yaml), for --shape
OTHER_SHAPES = {
    "xl": {"model_type": "gpt2", "n_layer": 48, "n_embd": 1600, "n_head": 25, "n_inner": 6400, "vocab_size": 50257,
           "n_positions": 1024, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"},
    "20b": {"model_type": "gpt2", "n_layer": 44, "n_embd": 6144, "n_head": 64, "n_inner": 24576, "vocab_size": 50257,
            "n_positions": 2048, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"},
}


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
    ap.add_argument("--prefill-len", type=int, default=2048, help="with --prefill-only: tokens of the prompt (the headline point is 2,048)")
    ap.add_argument("--shape", default="7b", choices=["7b", "xl", "20b"],
                    help="layer sizes of the decode workload: 7b is the headline's; xl and 20b measure the same step at the other "
                         "sizes of the reference's configurations (use --no-points: the prefill point is 2,048 tokens)")
    ap.add_argument("--workload", default="decode", choices=["decode", "xl_mix", "20b"],
                    help="decode: the workload described above. xl_mix / 20b: continuous-batching workloads at the gpt2_xl and gpt2_20b sizes "
                         "through InferenceEngine.generate; they print their own line")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py: this engine runs on one GPU; --gpus {args.gpus} is not supported")
        return 2

    import torch

    from levanter_amd.config import InferenceEngineConfig, LmConfig
    from levanter_amd.engine import InferenceEngine, Request

    if args.workload != "decode":
        return serving_workload(args)

    raw = load_baseline_config() if args.shape == "7b" else dict(OTHER_SHAPES[args.shape])
    shape_name = {"7b": "GPT-2 7B", "xl": "GPT-2 XL", "20b": "GPT-2 20B"}[args.shape]
    full_layers = raw["n_layer"]
    if args.layers is not None:
        raw["n_layer"] = args.layers
    cfg = LmConfig.from_dict(raw)
    ps = 16
    max_batch = max(args.batch, 1 if args.no_points else 64)
    # Requests whose prompts are done first decode beside the prompt portions of the others: `early` tokens at most
    # before the timed steps begin. Nobody may end, and no page may be missing, before the last timed step.
    early = (max_batch * args.prompt_len + 2047) // 2048 + 8
    # The timed steps lie in the middle of the GENERATED tokens that follow the prompt, however few they are: their mean
    # context is prompt_len + GENERATED / 2 (untimed steps lead up to them).
    span = max(args.steps, GENERATED)
    ctx_end = args.prompt_len + early + args.warmup + span + 1
    if ctx_end > cfg.n_positions:
        print(f"bench.py: prompt {args.prompt_len} + {early + args.warmup + span + 1} steps exceed n_positions {cfg.n_positions}")
        return 2
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
        reqs = [Request(prompt_tokens=p, request_id=i, max_new_tokens=early + warmup + max(steps, GENERATED) + 8, temperature=0.0)
                for i, p in enumerate(prompts(batch, args.prompt_len, seed))]
        seqs = engine.enqueue_requests(reqs)
        while any(s.n_cached < s.prompt_len for s in seqs) or any(not s.generated for s in seqs):
            engine.step()
        for _ in range(warmup):
            engine.step()
        ctx_now = sum(s.n_cached for s in seqs) / len(seqs)
        for _ in range(max(0, int(args.prompt_len + GENERATED / 2.0 - (steps + 1) / 2.0 - ctx_now))):
            engine.step()
        torch.cuda.synchronize()
        ctx0 = sum(s.n_cached for s in seqs) / len(seqs)
        before = dict(engine.stats)
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t = time.perf_counter()
        ev0.record()
        for _ in range(steps):
            engine.step()
        ev1.record()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t
        assert all(len(s.generated) >= warmup + steps and not s.done for s in seqs), "the timed steps did not all decode the whole batch"
        ctx_mean = ctx0 + (steps + 1) / 2.0
        # the device's own clock around the same steps, and the host's share of a step: what step() takes less the time it waits
        # for the device (src/levanter/inference/engine.py:1146-1159 logs the same split per iteration)
        timing = {"device_ms_per_step": round(ev0.elapsed_time(ev1) / steps, 4),
                  "host_ms_per_step": round(((engine.stats["step_s"] - before["step_s"]) - (engine.stats["wait_s"] - before["wait_s"])) / steps * 1e3, 4)}
        engine.reset()
        return dt, ctx_mean, timing

    def prefill_run(T, reps):
        """One prompt of T tokens in one step, ``reps`` times after one untimed run: the median, with the fastest and slowest."""
        times = []
        for rep in range(reps + 1):
            engine.reset()
            engine.enqueue_requests([Request(prompt_tokens=prompts(1, T, 50 + rep)[0], request_id=rep, max_new_tokens=1)])
            torch.cuda.synchronize()
            t = time.perf_counter()
            engine.step()
            torch.cuda.synchronize()
            if rep > 0:
                times.append(time.perf_counter() - t)
        times.sort()
        mid = times[len(times) // 2]
        flops = 2.0 * T * matrix_params + 2.0 * T * T * D * L + 2.0 * D * V
        return {"value": round(T / mid, 1), "tokens": T, "ms": round(mid * 1e3, 3), "frac": round(flops / mid / PEAK_FLOPS[args.dtype], 4),
                "ms_min": round(times[0] * 1e3, 3), "ms_max": round(times[-1] * 1e3, 3), "reps": reps}

    if args.prefill_only:
        if not 1 <= args.prefill_len < cfg.n_positions + 1:
            print(f"bench.py: --prefill-len {args.prefill_len} does not fit n_positions {cfg.n_positions}")
            return 2
        print(json.dumps({"prefill": prefill_run(args.prefill_len, 4), "model": f"gpt2_{args.shape} shape"}), flush=True)
        return 0

    dt, ctx_mean, timing = decode_run(args.batch, args.steps, args.warmup, seed=1)
    ms_per_step = dt / args.steps * 1e3
    value = args.batch * args.steps / dt
    step_bytes = weight_bytes + args.batch * ctx_mean * kv_bytes_per_token
    achieved = step_bytes / (dt / args.steps) / 1e9
    out = {
        "metric": (f"decode tok/s @ batch 8, {shape_name} shape, bf16" if args.batch == 8 and args.dtype == "bfloat16"
                   else f"decode tok/s @ batch {args.batch}, {shape_name} shape"),
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4), **timing, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "bf16" if args.dtype == "bfloat16" else "fp32", "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": f"gpt2_{args.shape} shape", "n_layer": L, "n_layer_full": full_layers, "n_embd": D, "n_head": cfg.n_head,
                   "head_dim": cfg.head_dim, "n_inner": F, "vocab_size": V, "n_positions": cfg.n_positions,
                   "global_batch": args.batch, "seq_len": args.prompt_len + GENERATED, "prompt_len": args.prompt_len,
                   "generated": GENERATED, "ctx_mean": round(ctx_mean, 1), "page_size": ps, "parallelism": "single GPU"},
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_BYTES_PER_S / 1e9, "unit": "GB/s",
                     "frac": round(achieved / (HBM_BYTES_PER_S / 1e9), 4)},
    }
    if not args.no_points:
        # prefill of one 2,048-token prompt in one step (the logits of its last token)
        out["prefill"] = prefill_run(2048, 5)
        points = {}
        for b, steps in ((1, min(args.steps, 128)), (64, min(args.steps, 64))):
            d, _, _ = decode_run(b, steps, min(args.warmup, 4), seed=2 + b)
            points[f"decode_b{b}"] = round(b * steps / d, 2)
        # the same prefill with every matrix product on this repository's own kernels (none left to the vendor library)
        kernels = engine.env.kernels
        was, kernels.gemm_library = kernels.gemm_library, False
        try:
            points["prefill_own_kernels"] = prefill_run(2048, 3)["value"]
        finally:
            kernels.gemm_library = was
        out["points"] = points
    print(json.dumps(out), flush=True)
    return 0


def serving_workload(args) -> int:
    """End-to-end generation through the scheduler: requests are admitted, their prompts cut into portions under the
    token budget beside the decoding requests, until every request has its tokens. One JSON line."""
    import torch

    from levanter_amd.config import InferenceEngineConfig, LmConfig
    from levanter_amd.engine import InferenceEngine, Request

    ps = 16
    if args.workload == "xl_mix":  # gpt2_xl sizes (config/gpt2_xl.yaml), 64 requests, prompts U[16, 768], 128 new tokens, portions of 256
        raw = {"model_type": "gpt2", "n_layer": 48, "n_embd": 1600, "n_head": 25, "n_inner": 6400, "vocab_size": 50257,
               "n_positions": 1024, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
        n_req, new_tokens, temperature, chunk = 64, 128, 0.0, 256
        g = torch.Generator().manual_seed(3)
        lens = torch.randint(16, 769, (n_req,), generator=g).tolist()
        name = "gpt2_xl shape, 64 requests, prompts U[16,768], 128 new tokens, portions of 256"
    else:  # gpt2_20b sizes (config/gpt2_20b.yaml), 32 requests x 1024-token prompts, 512 tokens each at temperature 1.0
        raw = {"model_type": "gpt2", "n_layer": 44, "n_embd": 6144, "n_head": 64, "n_inner": 24576, "vocab_size": 50257,
               "n_positions": 2048, "layer_norm_epsilon": 1e-5, "activation_function": "gelu_new"}
        n_req, new_tokens, temperature, chunk = 32, 512, 1.0, 2048
        lens = [1024] * n_req
        name = "gpt2_20b shape, 32 requests x 1024-token prompts, 512 new tokens at temperature 1.0"
    full_layers = raw["n_layer"]
    if args.layers is not None:
        raw["n_layer"] = args.layers
    cfg = LmConfig.from_dict(raw)
    V = cfg.vocab_size
    pages_per_seq = (max(lens) + new_tokens + ps) // ps
    itemsize = 2 if args.dtype == "bfloat16" else 4
    # 20b: the engine sizes the cache itself from what the weights leave of the memory (at most every request at full length)
    ecfg = InferenceEngineConfig(max_pages="auto" if args.workload == "20b" else n_req * pages_per_seq, cache_memory_reserve_gib=24.0,
                                 max_seqs=n_req, page_size=ps, max_pages_per_seq=pages_per_seq,
                                 compute_dtype=args.dtype, max_prefill_size=chunk, max_seqs_in_prefill=n_req, seed=0)
    t0 = time.time()
    engine = InferenceEngine.from_config(cfg, seed=0, config=ecfg)
    torch.cuda.synchronize()
    max_pages = max((g.pool.n_pages for g in engine.cache.groups), default=0)
    print(f"[bench] model ready in {time.time() - t0:.1f}s: {engine.model.weight_bytes() / 1e9:.2f} GB of weights, "
          f"{max_pages} pages of {ps} tokens", file=sys.stderr, flush=True)

    def requests(seed):
        g = torch.Generator().manual_seed(seed)
        return [Request(prompt_tokens=torch.randint(0, V, (n,), generator=g).tolist(), request_id=i, max_new_tokens=new_tokens,
                        temperature=temperature) for i, n in enumerate(lens)]

    # a short run first: kernels and the GEMM library are loaded (prompt portions of the workload's size among them) and
    # the decode shapes have been seen once
    warm = [Request(prompt_tokens=r.prompt_tokens[:chunk if i < 2 else 32], request_id=r.request_id, max_new_tokens=4, temperature=temperature)
            for i, r in enumerate(requests(1)[:4])]
    engine.generate(warm)
    engine.reset()
    engine.warm_up()
    step_ms = []
    print("[bench] warm-up done, the timed run starts", file=sys.stderr, flush=True)
    seqs = engine.enqueue_requests(requests(2))
    torch.cuda.synchronize()
    before = dict(engine.stats)
    t = time.perf_counter()
    while not all(s.done for s in seqs):
        t1 = time.perf_counter()
        engine.step()
        step_ms.append((time.perf_counter() - t1) * 1e3)
    torch.cuda.synchronize()
    dt = time.perf_counter() - t
    generated = sum(len(s.generated) for s in seqs)
    prompt_tokens = sum(lens)
    slowest = max(range(len(step_ms)), key=step_ms.__getitem__)
    print(f"[bench] {len(step_ms)} steps; the slowest was step {slowest} ({step_ms[slowest]:.1f} ms)", file=sys.stderr, flush=True)
    step_ms.sort()
    pick = lambda q: round(step_ms[min(len(step_ms) - 1, int(q * len(step_ms)))], 3)
    out = {
        "metric": f"end-to-end generated tok/s, {name}", "value": round(generated / dt, 2), "unit": "tok/s", "n_gpus": 1,
        "steps": len(step_ms), "warmup": 0, "ms_per_step": round(dt / len(step_ms) * 1e3, 4),
        "host_ms_per_step": round(((engine.stats["step_s"] - before["step_s"]) - (engine.stats["wait_s"] - before["wait_s"])) / len(step_ms) * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16" if args.dtype == "bfloat16" else "fp32",
        "data": "synthetic (random weights N(0,0.02), uniform-random token ids)",
        "config": {"model": args.workload, "n_layer": cfg.n_layer, "n_layer_full": full_layers, "n_embd": cfg.n_embd, "n_head": cfg.n_head,
                   "head_dim": cfg.head_dim, "n_inner": cfg.inner_dim, "vocab_size": V, "n_positions": cfg.n_positions,
                   "global_batch": n_req, "prompt_tokens": prompt_tokens, "new_tokens": new_tokens, "prefill_chunk": chunk,
                   "page_size": ps, "max_pages": max_pages, "temperature": temperature, "parallelism": "single GPU"},
        "seconds": round(dt, 3), "generated": generated, "all_tokens_per_s": round((generated + prompt_tokens) / dt, 1),
        "step_ms": {"p10": pick(0.1), "p50": pick(0.5), "p90": pick(0.9), "p99": pick(0.99), "max": round(step_ms[-1], 3)},
        "preemptions": engine.scheduler.n_preemptions,
    }
    print(json.dumps(out), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
