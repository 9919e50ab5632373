"""Causal self-attention over the paged cache, with any number of heads and key/value groups.

Reference formulas: the fused projection to (q, k, v) x heads x head_size
(src/levanter/models/gpt2.py:172-174,184-185), ``q / (layer_idx + 1)`` (gpt2.py:192-193) and the
scale 1/sqrt(head_size) (src/levanter/layers/attention.py:153-154), both folded into ``scale``
here; new keys and values go to their pages before attention, so a portion attends to itself
through the cache (attention.py:1559-1604, 1671-1699); scores, mask and softmax
(attention.py:347-378, paged: 1931-1981) run in 32-bit; then the output projection and the
residual sum (gpt2.py:211-212,240-242).
"""
from __future__ import annotations

from typing import Dict

import torch

from levanter_amd.cache.requirements import PagedKv
from .base import BuildEnv, CacheUnitView, Mixer, StepContext
from .embedding import tensors_of_nested
from .linear import Linear
from .registry import MIXERS, part_class
from .spec import PartSpec


@MIXERS.register("causal_self_attention")
class CausalSelfAttention(Mixer):
    graph_safe = True

    def __init__(self, spec: PartSpec, tensors: Dict[str, torch.Tensor], env: BuildEnv):
        super().__init__(spec, tensors, env)
        p = spec.params
        self.dim = int(p["dim"])
        self.n_heads = int(p["n_heads"])
        self.n_kv_heads = int(p["n_kv_heads"])
        self.head_dim = int(p["head_dim"])
        self.scale = float(p["scale"])
        self.window = p.get("window")
        # what a model may do to a score between the scaling and the mask (src/levanter/layers/attention.py:361-367): a
        # soft cap, and a term per head and distance from a float32 table [heads, distances] (the parameter ``score_bias``)
        self.softcap = p.get("softcap")
        bias = tensors.get("score_bias")
        self.score_bias = None if bias is None else bias.to(env.device, torch.float32).contiguous()
        if self.score_bias is not None and (self.score_bias.dim() != 2 or self.score_bias.shape[0] != self.n_heads):
            raise ValueError(f"attention: the score bias must be [heads={self.n_heads}, distances], got {tuple(self.score_bias.shape)}")
        if self.n_heads % self.n_kv_heads != 0:
            raise ValueError(f"attention: {self.n_heads} heads are not a multiple of {self.n_kv_heads} key/value heads")
        # the cache keeps keys in chunks of 8 head dimensions; the matrix-core kernels need multiples of 16
        step = 16 if env.dtype == torch.bfloat16 else 8
        if self.head_dim % step != 0:
            raise ValueError(f"attention: head_dim={self.head_dim} must be a multiple of {step} in {env.dtype}")
        layout = p.get("weight_layout", "out_in")
        self.qkv = Linear(tensors["qkv.weight"], tensors.get("qkv.bias"), layout, env)
        self.out = Linear(tensors["out.weight"], tensors.get("out.bias"), layout, env)
        self.q_cols = self.n_heads * self.head_dim
        self.kv_cols = self.n_kv_heads * self.head_dim
        if self.qkv.n_out != self.q_cols + 2 * self.kv_cols or self.qkv.n_in != self.dim:
            raise ValueError("attention: the fused projection does not have the sizes of the description")
        rotary = p.get("rotary")
        self.rotary = None
        if rotary is not None:
            self.rotary = part_class(rotary.kind, rotary.family or "position")(rotary, tensors_of_nested("rotary", tensors), env)
            self.graph_safe = bool(self.rotary.graph_safe)  # the rotation runs inside this mixer's forward

    def cache_requirement(self):
        return PagedKv(self.n_kv_heads, self.head_dim, self.window)

    def forward(self, h: torch.Tensor, x: torch.Tensor, ctx: StepContext, unit: CacheUnitView, writes_cache: bool) -> None:
        qkv = self.qkv(h, ctx)  # [T, (H + 2 KVH) * hd], compute dtype
        q = qkv[:, : self.q_cols]
        k = qkv[:, self.q_cols: self.q_cols + self.kv_cols]
        v = qkv[:, self.q_cols + self.kv_cols:]
        if self.rotary is not None:
            self.rotary.rotate(q, k, ctx)
        g = unit.group
        a = ctx.empty(h.shape[0], self.q_cols)
        args = dict(n_heads=self.n_heads, n_kv_heads=self.n_kv_heads, head_dim=self.head_dim, page_size=g.page_size,
                    scale=self.scale, window=self.window, block_tables=g.block_tables)
        if self.softcap or self.score_bias is not None:
            args.update(softcap=self.softcap, score_bias=self.score_bias)
        written = False
        if writes_cache:  # a step of single tokens writes the new keys and values inside the attention kernel
            written = ctx.kernels.paged_attention(q, a, unit.k_pages, unit.v_pages, ctx.attention, k_new=k, v_new=v,
                                                  dest=g.dest, **args)
        if not written:
            if writes_cache:
                ctx.kernels.kv_write(k, v, unit.k_pages, unit.v_pages, g.dest, self.n_kv_heads, self.head_dim, g.page_size)
            ctx.kernels.paged_attention(q, a, unit.k_pages, unit.v_pages, ctx.attention, **args)
        self.out(a, ctx, residual=x, final=True)
