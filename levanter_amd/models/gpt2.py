"""GPT-2 as a model description: which parts each layer has and where their tensors come from.

Reference: src/levanter/models/gpt2.py. Embeddings ``wte[token] + wpe[position]`` (:302-308);
each block is pre-LayerNorm (:237-248) with a fused-QKV multi-head attention (:158-214, columns
ordered q, k, v then heads then head_size, :172-174) and a two-matrix feed-forward (:132-155);
``ln_f`` after the last block (:271); the head is the token table (:361-362). Weights are
stored [in, out] (``out_first=False``, :142-143,172-177). Checkpoint names: ``wte``, ``wpe``
(:313-314), ``h.{i}`` (:275-276), an optional ``transformer.`` prefix (:80).
"""
from __future__ import annotations

import math

from levanter_amd.config.gpt2 import Gpt2Config
from levanter_amd.parts.spec import LayerSpec, ModelSpec, PartSpec, PlanEntry, TensorSpec


def gpt2_model_spec(cfg: Gpt2Config) -> ModelSpec:
    d, h, hd, f = cfg.n_embd, cfg.n_head, cfg.head_dim, cfg.inner_dim
    bias = cfg.use_bias

    def norm(prefix: str) -> PartSpec:
        tensors = {"weight": TensorSpec(prefix + ".weight", (d,), init="one_plus_normal")}
        if bias:
            tensors["bias"] = TensorSpec(prefix + ".bias", (d,))
        return PartSpec("layernorm", {"dim": d, "eps": cfg.layer_norm_epsilon, "bias": bias}, tensors, family="norm")

    def linear_tensors(prefix: str, n_in: int, n_out: int, local: str) -> dict:
        t = {local + ".weight": TensorSpec(prefix + ".weight", (n_in, n_out))}
        if bias:
            t[local + ".bias"] = TensorSpec(prefix + ".bias", (n_out,))
        return t

    layers = []
    for i in range(cfg.n_layer):
        p = f"h.{i}"
        # q / (layer_idx + 1) before the 1/sqrt(head_size) scale (gpt2.py:192-193; attention.py:153-154)
        scale = 1.0 / math.sqrt(hd)
        if cfg.scale_attn_by_inverse_layer_idx:
            scale = scale / (i + 1.0)
        mixer = PartSpec(
            "causal_self_attention",
            {
                "dim": d,
                "n_heads": h,
                "n_kv_heads": h,
                "head_dim": hd,
                "scale": scale,
                "window": None,
                "bias": bias,
                "weight_layout": "in_out",
                "rotary": None,
            },
            {**linear_tensors(p + ".attn.c_attn", d, 3 * d, "qkv"), **linear_tensors(p + ".attn.c_proj", d, d, "out")},
            family="mixer",
        )
        ff = PartSpec(
            "dense_mlp",
            {"dim": d, "inner_dim": f, "activation": cfg.activation_function, "bias": bias, "weight_layout": "in_out"},
            {**linear_tensors(p + ".mlp.c_fc", d, f, "up"), **linear_tensors(p + ".mlp.c_proj", f, d, "down")},
            family="feed_forward",
        )
        layers.append(LayerSpec("pre_norm", norm1=norm(p + ".ln_1"), mixer=mixer, norm2=norm(p + ".ln_2"), feed_forward=ff))

    position = PartSpec(
        "learned_absolute",
        {"n_positions": cfg.n_positions, "dim": d},
        {"table": TensorSpec("wpe.weight", (cfg.n_positions, d))},
        family="position",
    )
    embedding = PartSpec(
        "token_embedding",
        {"vocab_size": cfg.vocab_size, "dim": d, "position": position},
        {"table": TensorSpec("wte.weight", (cfg.vocab_size, d))},
        family="embedding",
    )
    head = PartSpec("tied_head", {"vocab_size": cfg.vocab_size, "dim": d}, {"table": TensorSpec("wte.weight", (cfg.vocab_size, d))},
                    family="head")
    return ModelSpec(
        architecture="gpt2",
        vocab_size=cfg.vocab_size,
        dim=d,
        embedding=embedding,
        layers=layers,
        plan=[PlanEntry(layer=i, cache=i, writes_cache=True) for i in range(cfg.n_layer)],
        final_norm=norm("ln_f"),
        head=head,
        max_positions=cfg.n_positions,
        strip_prefixes=("transformer.",),
        # the causal-mask buffers of GPT-2 checkpoints
        ignored_tensors=(r"h\.\d+\.attn\.bias", r"h\.\d+\.attn\.masked_bias"),
        # the head is the token table (gpt2.py:361-362): a stored head must be that table
        stored_copies={"lm_head.weight": "wte.weight"},
        init_std=cfg.initializer_range,
    )
