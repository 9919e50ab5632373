"""A plain, slow GPT-2 written from the reference's formulas: whole sequences, no cache.

One function per part; nothing here is shared with the engine. Every function cites the
place in the reference (paths relative to the reference checkout) whose formula it states.

Weights are a dict keyed by the checkpoint tensor names (``wte.weight``,
``h.0.attn.c_attn.weight`` ...), the configuration is the raw ``config.json`` dict.

``rounding`` lets a caller imitate a reduced-precision engine: it is applied where such an
engine stores an activation (after a norm, a projection, the activation function, the
attention probabilities and the attention output). The default is the identity.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional

import torch

Tensor = torch.Tensor
Rounding = Callable[[Tensor], Tensor]


def _identity(x: Tensor) -> Tensor:
    return x


def bf16_rounding(x: Tensor) -> Tensor:
    """Round to bfloat16 and return in the original dtype."""
    return x.to(torch.bfloat16).to(x.dtype)


# --------------------------------------------------------------------------- sizes


def plain_sizes(config: dict) -> dict:
    """Derived sizes. src/levanter/models/gpt2.py:66-72 (head size = hidden // heads; the
    reference's mlp width is hidden * 4, gpt2.py:43,71; ``n_inner`` overrides it here)."""
    d = int(config["n_embd"])
    h = int(config["n_head"])
    f = config.get("n_inner")
    return {
        "D": d,
        "H": h,
        "hd": d // h,
        "F": int(f) if f is not None else 4 * d,
        "L": int(config["n_layer"]),
        "V": int(config["vocab_size"]),
        "P": int(config["n_positions"]),
    }


# --------------------------------------------------------------------------- parts


def plain_embed(tokens: Tensor, positions: Tensor, wte: Tensor, wpe: Tensor) -> Tensor:
    """x[t] = wte[token_t] + wpe[pos_t]. src/levanter/models/gpt2.py:302-308 (dropout is 0)."""
    if int(tokens.min()) < 0 or int(tokens.max()) >= wte.shape[0]:
        raise IndexError("token id out of range")
    if int(positions.min()) < 0 or int(positions.max()) >= wpe.shape[0]:
        raise IndexError("position out of range")
    return wte[tokens] + wpe[positions]


def plain_layernorm(x: Tensor, weight: Tensor, bias: Optional[Tensor], eps: float) -> Tensor:
    """(x - mean) / sqrt(var + eps) * weight + bias over the last axis, biased variance.
    src/levanter/models/gpt2.py:228,230,263 (hnn.LayerNorm with eps=layer_norm_epsilon)."""
    mean = x.mean(dim=-1, keepdim=True)
    centered = x - mean
    var = (centered * centered).mean(dim=-1, keepdim=True)
    y = centered / torch.sqrt(var + eps) * weight
    if bias is not None:
        y = y + bias
    return y


def plain_activation(name: str) -> Callable[[Tensor], Tensor]:
    """src/levanter/utils/activation.py:18-40: gelu = exact erf form (:36), gelu_new = tanh
    approximation (:37), plus relu, silu/swish, quick_gelu, tanh."""

    def gelu_erf(u):
        return 0.5 * u * (1.0 + torch.erf(u / math.sqrt(2.0)))

    def gelu_tanh(u):
        return 0.5 * u * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (u + 0.044715 * u * u * u)))

    def silu(u):
        return u * torch.sigmoid(u)

    def quick_gelu(u):
        return u * torch.sigmoid(1.702 * u)

    table = {
        "gelu": gelu_erf,
        "gelu_new": gelu_tanh,
        "relu": torch.relu,
        "silu": silu,
        "swish": silu,
        "quick_gelu": quick_gelu,
        "tanh": torch.tanh,
    }
    return table[name]


def plain_linear(x: Tensor, weight_in_out: Tensor, bias: Optional[Tensor]) -> Tensor:
    """y = x @ W + b with W stored [in, out] (``out_first=False``).
    src/levanter/models/gpt2.py:142-143,172-177."""
    y = x @ weight_in_out
    if bias is not None:
        y = y + bias
    return y


def plain_split_qkv(qkv: Tensor, n_head: int) -> tuple:
    """Columns ordered (qkv=3, heads, head_size): [0:D]=Q, [D:2D]=K, [2D:3D]=V, head h at
    [h*hd:(h+1)*hd] inside each. src/levanter/models/gpt2.py:167-174,184-185. -> [H, T, hd] each."""
    t, three_d = qkv.shape
    d = three_d // 3
    hd = d // n_head
    parts = qkv.reshape(t, 3, n_head, hd)
    q, k, v = parts[:, 0], parts[:, 1], parts[:, 2]
    return q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1)


def plain_causal_attention(
    q: Tensor,
    k: Tensor,
    v: Tensor,
    *,
    q_offset: int = 0,
    scale: Optional[float] = None,
    window: Optional[int] = None,
    rounding: Rounding = _identity,
) -> Tensor:
    """softmax(mask(q*scale . k^T)) . v for [H, Tq, hd] queries over [H, Tk, hd] keys.

    src/levanter/layers/attention.py:347-378: the scale 1/sqrt(head_size) multiplies q
    (:353-356), masked scores are set to -1e9 (:370), softmax over keys (:372), the
    probabilities return to the activation dtype (:374) before the product with v (:378).
    Query row i stands at absolute position q_offset + i and sees keys j <= q_offset + i
    (the causal mask with an offset, attention.py:757-1050; used as kv_len - q_len in
    attention.py:1923). ``window`` (not used by GPT-2) keeps keys with position > query - window.
    """
    hd = q.shape[-1]
    if scale is None:
        scale = 1.0 / math.sqrt(hd)
    scores = (q * scale) @ k.transpose(-1, -2)  # [H, Tq, Tk]
    tq, tk = scores.shape[-2], scores.shape[-1]
    qpos = torch.arange(tq).unsqueeze(1) + q_offset
    kpos = torch.arange(tk).unsqueeze(0)
    allowed = kpos <= qpos
    if window is not None:
        allowed = allowed & (kpos > qpos - window)
    scores = torch.where(allowed, scores, torch.full_like(scores, -1e9))
    probs = torch.softmax(scores, dim=-1)
    probs = rounding(probs)
    return probs @ v


def plain_attention_layer(
    h: Tensor,
    weights: Dict[str, Tensor],
    prefix: str,
    config: dict,
    layer_idx: int,
    rounding: Rounding = _identity,
) -> Tensor:
    """c_attn -> split -> optional q / (layer_idx + 1) -> attention -> c_proj.
    src/levanter/models/gpt2.py:182-214 (the layer scale at :192-193, 0-based index :270)."""
    n_head = int(config["n_head"])
    qkv = rounding(plain_linear(h, weights[prefix + "attn.c_attn.weight"], weights.get(prefix + "attn.c_attn.bias")))
    q, k, v = plain_split_qkv(qkv, n_head)
    if config.get("scale_attn_by_inverse_layer_idx", False):
        q = q / (layer_idx + 1.0)
    o = plain_causal_attention(q, k, v, rounding=rounding)  # [H, T, hd]
    o = rounding(o.transpose(0, 1).reshape(h.shape[0], -1))  # heads, then head_size, flattened
    return plain_linear(o, weights[prefix + "attn.c_proj.weight"], weights.get(prefix + "attn.c_proj.bias"))


def plain_mlp(h: Tensor, weights: Dict[str, Tensor], prefix: str, config: dict, rounding: Rounding = _identity) -> Tensor:
    """c_proj(act(c_fc(h))). src/levanter/models/gpt2.py:150-155."""
    act = plain_activation(config.get("activation_function", "gelu_new"))
    m = plain_linear(h, weights[prefix + "mlp.c_fc.weight"], weights.get(prefix + "mlp.c_fc.bias"))
    m = rounding(act(m))
    return plain_linear(m, weights[prefix + "mlp.c_proj.weight"], weights.get(prefix + "mlp.c_proj.bias"))


def plain_block(x: Tensor, weights: Dict[str, Tensor], config: dict, layer_idx: int, rounding: Rounding = _identity) -> Tensor:
    """x + attn(ln_1(x)), then x + mlp(ln_2(x)). src/levanter/models/gpt2.py:237-248."""
    p = f"h.{layer_idx}."
    eps = float(config.get("layer_norm_epsilon", 1e-5))
    h = rounding(plain_layernorm(x, weights[p + "ln_1.weight"], weights.get(p + "ln_1.bias"), eps))
    x = x + plain_attention_layer(h, weights, p, config, layer_idx, rounding)
    h = rounding(plain_layernorm(x, weights[p + "ln_2.weight"], weights.get(p + "ln_2.bias"), eps))
    x = x + plain_mlp(h, weights, p, config, rounding)
    return x


def plain_hidden(weights: Dict[str, Tensor], config: dict, tokens: Tensor, positions: Optional[Tensor] = None,
                 rounding: Rounding = _identity) -> Tensor:
    """Embedding, the blocks in index order, ln_f. src/levanter/models/gpt2.py:345-359,268-273."""
    if positions is None:
        positions = torch.arange(tokens.shape[0])
    x = plain_embed(tokens, positions, weights["wte.weight"], weights["wpe.weight"])
    for layer_idx in range(int(config["n_layer"])):
        x = plain_block(x, weights, config, layer_idx, rounding)
    eps = float(config.get("layer_norm_epsilon", 1e-5))
    return rounding(plain_layernorm(x, weights["ln_f.weight"], weights.get("ln_f.bias"), eps))


def plain_logits(weights: Dict[str, Tensor], config: dict, tokens: Tensor, rounding: Rounding = _identity) -> Tensor:
    """logits[t, v] = sum_d ln_f(x)[t, d] * wte[v, d] (tied head).
    src/levanter/models/gpt2.py:361-362, src/levanter/models/lm_model.py:210. -> [T, V]."""
    hidden = plain_hidden(weights, config, tokens, rounding=rounding)
    return hidden @ weights["wte.weight"].T


# --------------------------------------------------------------------------- sampling


def plain_sample(logits: Tensor, temperature: float, gumbel: Optional[Tensor] = None) -> tuple:
    """src/levanter/layers/sampler.py:60-79: logits in 32-bit; greedy = argmax; otherwise a
    categorical draw from logits / temperature; the log-probability of the chosen token is
    scaled_logit - logsumexp(scaled_logits). A categorical draw is argmax(scaled + Gumbel
    noise); the noise is passed in so that the draw can be compared with the engine's."""
    logits = logits.to(torch.float32)
    if temperature == 0:
        token = int(torch.argmax(logits))
        scaled = logits
    else:
        scaled = logits / temperature
        token = int(torch.argmax(scaled + gumbel))
    logprob = float(scaled[token] - torch.logsumexp(scaled, dim=-1))
    return token, logprob


def plain_greedy_generate(weights: Dict[str, Tensor], config: dict, prompt: List[int], n_new: int,
                          rounding: Rounding = _identity) -> List[int]:
    """Greedy continuation by running the whole sequence again for every new token."""
    tokens = list(prompt)
    out = []
    for _ in range(n_new):
        logits = plain_logits(weights, config, torch.tensor(tokens, dtype=torch.long), rounding)
        nxt = int(torch.argmax(logits[-1].to(torch.float32)))
        out.append(nxt)
        tokens.append(nxt)
    return out


def plain_is_stop(tail: List[int], stop_sequences: List[List[int]]) -> bool:
    """True if the generated tokens end with one of the stop sequences; an empty sequence
    never matches. src/levanter/inference/utils.py:46-64 (left-padded compare)."""
    for seq in stop_sequences:
        n = len(seq)
        if n == 0 or n > len(tail):
            continue
        if list(tail[-n:]) == list(seq):
            return True
    return False


# --------------------------------------------------------------------------- random weights


def plain_random_weights(config: dict, seed: int, dtype=torch.float64) -> Dict[str, Tensor]:
    """Independent random weights for tests of this file alone (not the engine's generator):
    matrices and biases N(0, 0.02), norm weights 1 + N(0, 0.02)."""
    s = plain_sizes(config)
    g = torch.Generator().manual_seed(seed)

    def n(*shape):
        return (torch.randn(*shape, generator=g, dtype=torch.float64) * 0.02).to(dtype)

    w = {"wte.weight": n(s["V"], s["D"]), "wpe.weight": n(s["P"], s["D"])}
    for i in range(s["L"]):
        p = f"h.{i}."
        w[p + "ln_1.weight"] = 1 + n(s["D"])
        w[p + "ln_1.bias"] = n(s["D"])
        w[p + "attn.c_attn.weight"] = n(s["D"], 3 * s["D"])
        w[p + "attn.c_attn.bias"] = n(3 * s["D"])
        w[p + "attn.c_proj.weight"] = n(s["D"], s["D"])
        w[p + "attn.c_proj.bias"] = n(s["D"])
        w[p + "ln_2.weight"] = 1 + n(s["D"])
        w[p + "ln_2.bias"] = n(s["D"])
        w[p + "mlp.c_fc.weight"] = n(s["D"], s["F"])
        w[p + "mlp.c_fc.bias"] = n(s["F"])
        w[p + "mlp.c_proj.weight"] = n(s["F"], s["D"])
        w[p + "mlp.c_proj.bias"] = n(s["D"])
    w["ln_f.weight"] = 1 + n(s["D"])
    w["ln_f.bias"] = n(s["D"])
    return w
