"""InferenceEngine: the Python entry point. From requests to generated tokens.

Reference: ``InferenceEngine.from_model_with_config`` / ``.generate(requests) -> GenerationResult``
/ ``.reset()`` (src/levanter/inference/engine.py:705-776,1019-1199). Returned tokens are the
generated ones only, the stopping token included (engine.py:613,
tests/inference/test_engine.py:87-92), ordered by request and generation (engine.py:1173-1190).
"""
from __future__ import annotations

import logging
import time
from typing import List, Optional, Sequence

import torch

from levanter_amd.config import InferenceEngineConfig, LmConfig
from levanter_amd.parts import BuildEnv, DecoderLm
from levanter_amd.sampling import Sampler, fold_in, make_key

from .loading import load_model, make_cache, make_env, random_model
from .request import GenerationResult, Request, SeqDecodingParams
from .scheduler import PlannedEntry, Scheduler, Sequence_
from .step import ModelRunner, StepEntry

logger = logging.getLogger(__name__)

__all__ = ["InferenceEngine", "Request", "SeqDecodingParams", "GenerationResult", "InferenceEngineConfig"]


class _Launched:
    """A step that runs on the GPU: its plan, its sampling under way, and whether its sampled tokens can feed the
    next step on the device (every entry one decoded token that wants logits)."""

    def __init__(self, plan, sample):
        self.plan, self.sample = plan, sample


class InferenceEngine:
    def __init__(self, model, config: InferenceEngineConfig, env: BuildEnv, allocate: bool = True):
        self.model = model
        self.config = config
        self.env = env
        self.cache = make_cache(model, config, env)
        self.runner = ModelRunner(model, self.cache, env, allocate=allocate)
        self.sampler = Sampler(env.kernels, env.device)
        self.scheduler = Scheduler(self.cache, config, self.runner.max_len)
        # launch_s: the host's time to plan tables and launch kernels; wait_s: the time it then waited for the device (the copy
        # of the sampled tokens); step_s: all of step(). The host's own share of a step is step_s - wait_s, as the reference
        # logs it per iteration (src/levanter/inference/engine.py:1146-1159: host = total - device wait).
        self.stats = {"steps": 0, "commits": 0, "tokens_in": 0, "launch_s": 0.0, "wait_s": 0.0, "step_s": 0.0}
        self._pending: Optional[_Launched] = None  # a step launched ahead of the one being committed

    # ---- construction -------------------------------------------------------------------------
    @classmethod
    def from_pretrained(cls, model_dir: str, config: Optional[InferenceEngineConfig] = None, device: Optional[str] = None):
        """Load ``config.json`` and ``model.safetensors`` of a folder; the architecture comes from the registry."""
        config = config or InferenceEngineConfig()
        env = make_env(config.compute_dtype, device)
        _, model = load_model(model_dir, env)
        return cls(model, config, env)

    @classmethod
    def from_config(cls, model_config: LmConfig, seed: int = 0, config: Optional[InferenceEngineConfig] = None,
                    device: Optional[str] = None):
        """A model with random weights drawn on the GPU from ``seed``."""
        config = config or InferenceEngineConfig()
        env = make_env(config.compute_dtype, device)
        return cls(random_model(model_config, seed, env), config, env)

    @classmethod
    def from_model_with_config(cls, model: DecoderLm, tokenizer=None, config: Optional[InferenceEngineConfig] = None):
        """The reference's constructor name (engine.py:705-731); the tokenizer is not needed: token ids in and out."""
        return cls(model, config or InferenceEngineConfig(), model.env)

    @classmethod
    def from_model(cls, model: DecoderLm, tokenizer=None, *, max_pages, max_seqs: int, page_size: int, max_pages_per_seq: int,
                   compute_dtype=None, max_queued_tokens: int = 32, max_seqs_in_prefill: int = 16, max_prefill_size: Optional[int] = None):
        """The reference's constructor from sizing arguments (engine.py:705-731). ``compute_dtype`` is the cache's dtype and
        must be the dtype the model was built in (left out: that one)."""
        built = {torch.bfloat16: "bfloat16", torch.float32: "float32"}[model.env.dtype]
        name = built if compute_dtype is None else {torch.bfloat16: "bfloat16", torch.float32: "float32"}.get(compute_dtype, compute_dtype)
        if name != built:
            raise ValueError(f"from_model: the model was built in {built}, the cache cannot be {name}")
        return cls.from_model_with_config(model, tokenizer, InferenceEngineConfig(
            max_pages=max_pages, max_seqs=max_seqs, page_size=page_size, max_pages_per_seq=max_pages_per_seq, compute_dtype=name,
            max_queued_tokens=max_queued_tokens, max_seqs_in_prefill=max_seqs_in_prefill, max_prefill_size=max_prefill_size))

    # ---- requests ---------------------------------------------------------------------------------
    def _validate(self, requests: Sequence[Request]) -> None:
        cfg = self.config
        v = self.model.vocab_size
        for r in requests:
            if r.n_generations < 1 or r.n_generations > cfg.max_seqs:
                raise ValueError(f"request {r.request_id}: n_generations={r.n_generations} must be in 1..max_seqs={cfg.max_seqs}")
            if len(r.prompt_tokens) == 0:
                raise ValueError(f"request {r.request_id}: empty prompt")
            if len(r.prompt_tokens) > self.runner.max_len:
                raise ValueError(f"request {r.request_id}: a prompt of {len(r.prompt_tokens)} tokens is longer than the "
                                 f"limit of {self.runner.max_len} (model positions and page_size * max_pages_per_seq)")
            bad = [t for t in r.prompt_tokens if not 0 <= t < v]
            if bad:
                raise ValueError(f"request {r.request_id}: token id {bad[0]} is outside the vocabulary of {v}")
            stops = r.decode_params.stop_tokens
            if stops is not None:
                if len(stops) > cfg.max_stop_seqs:
                    raise ValueError(f"request {r.request_id}: {len(stops)} stop sequences, max_stop_seqs={cfg.max_stop_seqs}")
                if any(len(s) > cfg.max_stop_tokens for s in stops):
                    raise ValueError(f"request {r.request_id}: a stop sequence is longer than max_stop_tokens={cfg.max_stop_tokens}")
            if r.enable_logprobs and not cfg.enable_logprobs:
                raise ValueError(f"request {r.request_id} asks for logprobs but the engine has enable_logprobs=False")

    def enqueue_requests(self, requests: Sequence[Request]) -> List[Sequence_]:
        self._validate(requests)
        seqs = []
        for r in requests:
            k = r.decode_params.key
            base = fold_in(make_key(self.config.seed), r.request_id) if k is None else (make_key(k) if isinstance(k, int) else tuple(k))
            for child in range(r.n_generations):
                key = base if r.n_generations == 1 else fold_in(base, child)
                seq = Sequence_(request=r, child=child, key=key, order=self.scheduler.next_order(),
                                tokens=list(r.prompt_tokens), prompt_len=len(r.prompt_tokens))
                self.scheduler.add(seq)
                seqs.append(seq)
        return seqs

    # ---- one scheduler iteration -----------------------------------------------------------------------
    def step(self) -> List[Sequence_]:
        """Commit one step: plan it and run it (unless it was launched ahead already), sample, append the tokens.
        Returns the sequences that finished in it.

        Steps are pipelined: while the GPU runs a step, the step after it is planned from what the host knows
        (prompt portions, admissions, which requests will decode) and launched with the decoded token ids taken from
        the sampler's output on the device, and only then are the first step's tokens read back. The GPU does not wait
        for the host between steps. What cannot be known without the tokens (a stop sequence that ends a request) is
        settled afterwards: the request's row of the step launched ahead is ignored, and what that row wrote lies in
        pages that its request no longer owns and nobody reads."""
        t_step = time.perf_counter()
        debug = logger.isEnabledFor(logging.DEBUG)
        before = dict(self.stats) if debug else None
        try:
            return self._step()
        finally:
            dt = time.perf_counter() - t_step
            self.stats["step_s"] += dt
            if debug:  # the reference logs every decode iteration's device and host time (engine.py:1146-1159)
                wait = self.stats["wait_s"] - before["wait_s"]
                logger.debug("step: %.3f ms (waiting for the GPU %.3f ms, host %.3f ms of which planning and launching %.3f ms), "
                             "%d tokens in", 1e3 * dt, 1e3 * wait, 1e3 * (dt - wait), 1e3 * (self.stats["launch_s"] - before["launch_s"]),
                             self.stats["tokens_in"] - before["tokens_in"])

    def _read(self, sample):
        t0 = time.perf_counter()
        out = self.sampler.read(sample)
        self.stats["wait_s"] += time.perf_counter() - t0
        return out

    def _step(self) -> List[Sequence_]:
        pend = self._pending
        self._pending = None
        if pend is None:
            plan: List[PlannedEntry] = self.scheduler.plan()
            if not plan:
                return []
            pend = self._launch(plan, None)
        self.stats["commits"] += 1
        nxt = None
        if self.config.decode_lookahead:
            ahead = self.scheduler.plan_lookahead(pend.plan)
            if ahead is not None:
                nxt = self._launch(ahead[0], (pend.sample.tokens, ahead[1]) if ahead[1] else None)
        toks, lps = ([], []) if pend.sample is None else self._read(pend.sample)
        finished = self.scheduler.commit(pend.plan, toks, lps)
        if nxt is not None:
            if all(e.seq.done for e in nxt.plan):  # every request of the step launched ahead has ended meanwhile
                if nxt.sample is not None:
                    self.sampler.read(nxt.sample)
            else:
                self._pending = nxt
        return finished

    def _launch(self, plan: List[PlannedEntry], feed) -> "_Launched":
        """Run a planned step and start sampling; nothing is waited for. ``feed = (device tokens, rows)``: the
        entries' tokens are the sampled tokens of the step before, still on the device."""
        entries = [StepEntry(e.seq.handle, e.tokens, [len(e.tokens) - 1] if e.wants_logits else []) for e in plan]
        t0 = time.perf_counter()
        token_feed = None
        if feed is not None:
            device_tokens, rows = feed
            same = rows == list(range(len(rows))) and len(rows) == int(device_tokens.numel())
            token_feed = (device_tokens, None if same else torch.tensor(rows, dtype=torch.int32, device=device_tokens.device), len(rows))
        logits = self.runner.step(entries, copy_out=False, token_feed=token_feed)
        wanted = [e for e in plan if e.wants_logits]
        sample = None
        if wanted:
            temps = [e.seq.request.decode_params.temperature for e in wanted]
            keys = [e.seq.key for e in wanted]
            positions = [e.seq.n_cached - 1 for e in wanted]  # position of the token whose logits are sampled
            sample = self.sampler.launch(logits, temps, keys, positions)
        self.stats["steps"] += 1
        self.stats["tokens_in"] += sum(len(e.tokens) for e in plan)
        self.stats["launch_s"] += time.perf_counter() - t0  # the host's time to plan the tables and launch the kernels
        return _Launched(plan, sample)

    def generate(self, requests: Sequence[Request]) -> GenerationResult:
        seqs = self.enqueue_requests(requests)
        t0 = time.perf_counter()
        stats0 = dict(self.stats)
        idle_steps = 0
        while not all(s.done for s in seqs):
            # progress: a step was launched, a step launched earlier was committed, or a sequence ended (the planner
            # ends a lone sequence that the pool cannot hold without launching anything)
            before = (self.stats["steps"], self.stats["commits"], sum(s.done for s in seqs))
            self.step()
            idle_steps = idle_steps + 1 if (self.stats["steps"], self.stats["commits"], sum(s.done for s in seqs)) == before else 0
            if idle_steps >= 2:  # the reference breaks after two iterations without progress (engine.py:1160-1171)
                raise RuntimeError("the scheduler made no step twice in a row although requests are unfinished")
        dt = time.perf_counter() - t0
        total = sum(len(s.generated) for s in seqs)
        wait = self.stats["wait_s"] - stats0["wait_s"]
        logger.info("generated %d tokens in %.3fs (%.1f tok/s): %d steps, waiting for the GPU %.3fs, host %.3fs", total, dt,
                    total / max(dt, 1e-9), self.stats["steps"] - stats0["steps"], wait, max(dt - wait, 0.0))
        want_lp = self.config.enable_logprobs and any(s.request.enable_logprobs for s in seqs)
        return GenerationResult(tokens=[list(s.generated) for s in seqs],
                                logprobs=[list(s.logprobs) for s in seqs] if want_lp else None,
                                total_generated=total, finish_reasons=[s.finish_reason for s in seqs])

    def warm_up(self, token_counts: Optional[Sequence[int]] = None) -> None:
        """Run prompts of several lengths once and drop them: kernels, and the GEMM library's code for the row counts
        that prompt portions, decode batches and mixed steps will have, are loaded and timed before the first request is
        (a first use can take a fifth of a second). ``token_counts``: prompt tokens of each warm-up step; default: a ladder
        from 32 up to ``max_prefill_size``. A step may hold more prompt tokens than one request can (the budget is the
        step's, the length limit the request's): such a count is made of several requests that are admitted together."""
        one = self.runner.max_len - 1  # the longest prompt that still generates a token
        budget = self.config.imputed_max_prefill_size
        most = self.config.max_seqs
        limit = min(budget, one * min(most, self.config.max_seqs_in_prefill))
        if token_counts is None:
            token_counts = [n for n in (32, 64, 128, 192, 256, 288, 320, 384, 448, 512, 640, 768, 1024, 1280, 1536, 2048) if n <= limit]
            for n in (min(budget, one), limit):
                if n not in token_counts:
                    token_counts.append(n)
        if not self.scheduler.idle or self._pending is not None:
            raise RuntimeError("warm_up() runs on an idle engine")
        v = self.model.vocab_size

        def prompts(n: int, first_id: int) -> List[Request]:
            """Requests whose prompts have n tokens together, each as long as a request may be but the last."""
            out = []
            while n > 0:
                k = min(n, one)
                out.append(Request(prompt_tokens=[(7 * i + 3) % v for i in range(k)], request_id=first_id - len(out), max_new_tokens=1))
                n -= k
            return out

        for n in token_counts:
            self.generate(prompts(max(1, min(int(n), limit)), -1))
            self.reset()
        # batches of decoding requests: the head and the products of a decode step at the row counts where the library takes them
        for b in sorted({b for b in (most, most // 2, 48, 32, 25) if 25 <= b <= most}):
            self.generate([Request(prompt_tokens=[(3 * i + 1) % v], request_id=-1 - i, max_new_tokens=3) for i in range(b)])
        # a whole step's worth of prompt tokens beside decoding requests: the row counts of mixed steps, which are no multiple
        # of anything (the library keeps the kernel it timed fastest for row counts up to the same multiple of 64; timing
        # takes a fifth of a second at 20B sizes)
        rounds = self.config.max_rounds  # decode steps that may pass before a waiting request is admitted
        from .step import MIXED_DECODE_BUCKET

        # one run for every number of single tokens that such steps are filled up to, with prompt tokens for two full steps:
        # a shape that has come twice is recorded and replayed from then on
        for d in sorted({min(d, most - 1) for d in range(1, most, MIXED_DECODE_BUCKET)}):
            self.enqueue_requests([Request(prompt_tokens=[(3 * i + 1) % v], request_id=-1 - i, max_new_tokens=rounds + 8) for i in range(d)])
            self.step()
            self.enqueue_requests(prompts(min(2 * limit, one * max(1, min(most - d, self.config.max_seqs_in_prefill))), -1 - d))
            for _ in range(rounds + 12):
                if self.scheduler.idle and self._pending is None:
                    break
                self.step()
            self.reset()
        self.reset()

    def reset(self) -> None:
        """Drop every request and give back all pages and slots (engine.py:761-776)."""
        if self._pending is not None and self._pending.sample is not None:
            self.sampler.read(self._pending.sample)  # let the step launched ahead finish before its pages go
        self._pending = None
        self.scheduler.abort_all()
        self.cache.reset()
