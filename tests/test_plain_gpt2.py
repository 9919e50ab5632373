"""Pins the plain implementation by what fixes it beside the reference's text: library
routines it must reduce to, vectors the reference's own tests hold, and invariants. Each
check is chosen so that a plausible mistake fails it."""
import math

import pytest
import torch
import torch.nn.functional as F

import plain_gpt2 as P
from tiny_configs import TINY_A, TINY_B

torch.manual_seed(0)
D64 = torch.float64


def test_layernorm_is_library_layer_norm():
    x = torch.randn(5, 96, dtype=D64) * 3 + 1.5
    w = torch.randn(96, dtype=D64)
    b = torch.randn(96, dtype=D64)
    for eps in (1e-5, 1e-6, 0.1):  # a large eps shows an eps outside the root
        torch.testing.assert_close(P.plain_layernorm(x, w, b, eps), F.layer_norm(x, (96,), w, b, eps), rtol=1e-12, atol=1e-12)
    # a constant row has variance 0: the output is exactly the bias
    const = torch.full((1, 96), 7.0, dtype=D64)
    torch.testing.assert_close(P.plain_layernorm(const, w, b, 1e-5), b.unsqueeze(0))
    # shift invariance
    torch.testing.assert_close(P.plain_layernorm(x + 11.0, w, b, 1e-5), P.plain_layernorm(x, w, b, 1e-5), rtol=1e-9, atol=1e-9)


def test_activations_are_the_library_ones_and_not_each_other():
    u = torch.linspace(-6, 6, 241, dtype=D64)
    torch.testing.assert_close(P.plain_activation("gelu")(u), F.gelu(u), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(P.plain_activation("gelu_new")(u), F.gelu(u, approximate="tanh"), rtol=1e-12, atol=1e-12)
    torch.testing.assert_close(P.plain_activation("silu")(u), F.silu(u))
    torch.testing.assert_close(P.plain_activation("swish")(u), F.silu(u))
    torch.testing.assert_close(P.plain_activation("relu")(u), F.relu(u))
    # u sigmoid(a u) = silu(a u) / a: quick_gelu through the library's silu
    torch.testing.assert_close(P.plain_activation("quick_gelu")(u), F.silu(1.702 * u) / 1.702, rtol=1e-12, atol=1e-12)
    assert float((P.plain_activation("quick_gelu")(u) - F.gelu(u)).abs().max()) > 1e-3  # and it is not a gelu
    # the two gelus differ where |u| is about 2: a swapped option cannot pass both checks above
    diff = (P.plain_activation("gelu")(u) - P.plain_activation("gelu_new")(u)).abs().max()
    assert 1e-4 < float(diff) < 1e-2
    for name in ("gelu", "gelu_new"):
        act = P.plain_activation(name)
        assert float(act(torch.tensor(0.0, dtype=D64))) == 0.0
        assert abs(float(act(torch.tensor(-10.0, dtype=D64)))) < 1e-6
        assert abs(float(act(torch.tensor(10.0, dtype=D64))) - 10.0) < 1e-6


def test_linear_layout_is_in_out():
    x = torch.randn(3, 8, dtype=D64)
    w = torch.randn(8, 8, dtype=D64)  # square and asymmetric: a transposed read differs
    b = torch.randn(8, dtype=D64)
    torch.testing.assert_close(P.plain_linear(x, w, b), torch.addmm(b, x, w))
    assert not torch.allclose(P.plain_linear(x, w, b), torch.addmm(b, x, w.T))
    w2 = torch.randn(8, 20, dtype=D64)  # not square: a transposed read fails by shape
    assert P.plain_linear(x, w2, None).shape == (3, 20)


def test_qkv_roles_and_head_columns_through_library_attention():
    """Which third of the fused projection is the query, the key and the value, and which columns are a head. The
    order (q, k, v), then heads, then head size is the reference's (src/levanter/models/gpt2.py:172-174,184-185 with
    the flattening of src/levanter/compat/hf_checkpoints.py); no stored numbers of the reference cover it, so against
    another implementation this order is "parity unpinned". What is pinned: each third plays its role. With the first
    third's weight zero and its bias a constant vector c, every query is c: scores depend on the key only, and the
    result is the library's attention with q = c. Were the first third the keys, scores would not depend on the key
    and every row would be a running mean of the values; were it the values, the output would be c."""
    n_head, hd, t = 3, 32, 7
    d = n_head * hd
    g = torch.Generator().manual_seed(11)
    h = torch.randn(t, d, dtype=D64, generator=g)
    w = torch.randn(d, 3 * d, dtype=D64, generator=g) * 0.3
    b = torch.randn(3 * d, dtype=D64, generator=g)
    c = torch.randn(d, dtype=D64, generator=g) * 2
    w[:, :d] = 0
    b[:d] = c
    q, k, v = P.plain_split_qkv(P.plain_linear(h, w, b), n_head)
    got = P.plain_causal_attention(q, k, v)
    heads = lambda m: m.reshape(t, n_head, hd).transpose(0, 1)  # columns of a third: head-major
    want = F.scaled_dot_product_attention(heads(c.expand(t, d)), heads(h @ w[:, d:2 * d] + b[d:2 * d]),
                                          heads(h @ w[:, 2 * d:] + b[2 * d:]), is_causal=True)
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-10)
    running_mean = torch.cumsum(heads(h @ w[:, 2 * d:] + b[2 * d:]), 1) / torch.arange(1, t + 1, dtype=D64).view(1, t, 1)
    assert not torch.allclose(got, running_mean, atol=1e-3)
    # the last third is the value: with it zero (weight and bias) the output vanishes whatever q and k are
    w2, b2 = w.clone(), b.clone()
    w2[:, 2 * d:] = 0
    b2[2 * d:] = 0
    q, k, v = P.plain_split_qkv(P.plain_linear(h, w2, b2), n_head)
    assert float(P.plain_causal_attention(q, k, v).abs().max()) == 0.0
    # head-major columns inside a third: the split of a counted matrix
    qkv = torch.arange(t * 3 * d, dtype=D64).reshape(t, 3 * d)
    q, k, v = P.plain_split_qkv(qkv, n_head)
    assert q.shape == (n_head, t, hd)
    torch.testing.assert_close(k[2, 4], qkv[4, 1 * d + 2 * hd: 1 * d + 3 * hd])


def test_attention_is_library_sdpa():
    h, t, hd = 3, 11, 32
    q, k, v = (torch.randn(h, t, hd, dtype=D64) for _ in range(3))
    want = F.scaled_dot_product_attention(q, k, v, is_causal=True)
    torch.testing.assert_close(P.plain_causal_attention(q, k, v), want, rtol=1e-10, atol=1e-10)
    # one head, and a scale that folds a layer index in
    want = F.scaled_dot_product_attention(q[:1], k[:1], v[:1], is_causal=True, scale=1 / (math.sqrt(hd) * 3))
    torch.testing.assert_close(P.plain_causal_attention(q[:1] / 3.0, k[:1], v[:1]), want, rtol=1e-10, atol=1e-10)
    # first row sees only the first key: its output is v[0]
    torch.testing.assert_close(P.plain_causal_attention(q, k, v)[:, 0], v[:, 0], rtol=1e-10, atol=1e-10)


def test_attention_offset_equals_rows_of_full_causal():
    # the vector of the reference's tests/test_attention.py:415-487: 6 keys, the last 2 queries
    # with offset 4 give rows 4:6 of full causal attention; without the offset they do not.
    h, t, hd = 2, 6, 4
    q, k, v = (torch.randn(h, t, hd, dtype=D64) for _ in range(3))
    full = P.plain_causal_attention(q, k, v)
    part = P.plain_causal_attention(q[:, 4:6], k, v, q_offset=4)
    torch.testing.assert_close(part, full[:, 4:6], rtol=1e-12, atol=1e-12)
    wrong = P.plain_causal_attention(q[:, 4:6], k, v, q_offset=0)
    assert not torch.allclose(wrong, full[:, 4:6], atol=2e-3)


def test_attention_window_and_shift_of_positions():
    h, t, hd = 2, 12, 16
    q, k, v = (torch.randn(h, t, hd, dtype=D64) for _ in range(3))
    w = 4
    got = P.plain_causal_attention(q, k, v, window=w)
    mask = torch.ones(t, t, dtype=torch.bool).tril() & ~torch.ones(t, t, dtype=torch.bool).tril(-w)
    want = F.scaled_dot_product_attention(q, k, v, attn_mask=mask)
    torch.testing.assert_close(got, want, rtol=1e-10, atol=1e-10)
    # only distances count inside attention: the last rows over the last keys equal a shifted problem
    a = P.plain_causal_attention(q[:, 8:], k[:, 5:], v[:, 5:], q_offset=3, window=w)
    torch.testing.assert_close(a, got[:, 8:], rtol=1e-10, atol=1e-10)


def test_embedding_positions_are_absolute():
    wte = torch.randn(50, 8, dtype=D64)
    wpe = torch.randn(16, 8, dtype=D64)
    toks = torch.randint(0, 50, (10,))
    whole = P.plain_embed(toks, torch.arange(10), wte, wpe)
    part = P.plain_embed(toks[5:], torch.arange(5, 10), wte, wpe)
    torch.testing.assert_close(part, whole[5:])
    with pytest.raises(IndexError):
        P.plain_embed(torch.tensor([50]), torch.tensor([0]), wte, wpe)
    with pytest.raises(IndexError):
        P.plain_embed(torch.tensor([1]), torch.tensor([16]), wte, wpe)


@pytest.mark.parametrize("config,seed", [(TINY_A, 0), (TINY_B, 1)])
def test_whole_model_shapes_causality_and_tied_head(config, seed):
    w = P.plain_random_weights(config, seed)
    s = P.plain_sizes(config)
    assert w["h.0.mlp.c_fc.weight"].shape == (s["D"], s["F"])
    toks = torch.randint(0, s["V"], (19,), generator=torch.Generator().manual_seed(5))
    logits = P.plain_logits(w, config, toks)
    assert logits.shape == (19, s["V"])
    # causality: a later token does not change earlier logits
    toks2 = toks.clone()
    toks2[12] = (toks2[12] + 1) % s["V"]
    logits2 = P.plain_logits(w, config, toks2)
    torch.testing.assert_close(logits2[:12], logits[:12], rtol=1e-12, atol=1e-12)
    assert not torch.allclose(logits2[12:], logits[12:])
    # the head is the token table (src/levanter/models/gpt2.py:361-362): changing the row of a token that is not in the
    # prompt changes nothing before the head, so exactly that token's logits move, by hidden . delta
    absent = next(v for v in range(s["V"]) if v not in set(toks.tolist()))
    w3 = dict(w)
    delta = torch.linspace(-1, 1, s["D"], dtype=w["wte.weight"].dtype)
    w3["wte.weight"] = w["wte.weight"].clone()
    w3["wte.weight"][absent] += delta
    logits3 = P.plain_logits(w3, config, toks)
    moved = (logits3 - logits).abs().max(0).values
    assert float(moved[absent]) > 1e-3
    moved[absent] = 0
    assert float(moved.max()) == 0.0
    torch.testing.assert_close(logits3[:, absent] - logits[:, absent], P.plain_hidden(w, config, toks) @ delta, rtol=1e-9, atol=1e-9)


def test_pre_norm_placement_and_layer_scale():
    # with the attention and mlp output projections zeroed, blocks are the identity: x passes
    # through unchanged and the logits are ln_f(embedding) @ wte^T. A post-norm block would differ.
    config = dict(TINY_B)
    w = P.plain_random_weights(config, 3)
    for i in range(config["n_layer"]):
        for name in ("attn.c_proj", "mlp.c_proj"):
            w[f"h.{i}.{name}.weight"].zero_()
            w[f"h.{i}.{name}.bias"].zero_()
    toks = torch.tensor([3, 1, 4, 1, 5])
    x = P.plain_embed(toks, torch.arange(5), w["wte.weight"], w["wpe.weight"])
    want = F.layer_norm(x, (96,), w["ln_f.weight"], w["ln_f.bias"], 1e-6) @ w["wte.weight"].T
    torch.testing.assert_close(P.plain_logits(w, config, toks), want, rtol=1e-10, atol=1e-10)
    # layer scale: q / (layer_idx + 1) changes layers after the first only
    w = P.plain_random_weights(config, 4)
    for k in w:
        if "c_attn" in k:
            w[k] = w[k] * 30  # make attention sharp enough for the scale to matter
    h = torch.randn(7, 96, dtype=D64)
    off = dict(config, scale_attn_by_inverse_layer_idx=False)
    torch.testing.assert_close(P.plain_attention_layer(h, w, "h.0.", config, 0), P.plain_attention_layer(h, w, "h.0.", off, 0))
    assert not torch.allclose(P.plain_attention_layer(h, w, "h.1.", config, 1), P.plain_attention_layer(h, w, "h.1.", off, 1))


def test_zeroing_one_heads_query_columns_changes_only_that_head():
    config = dict(TINY_B)
    w = P.plain_random_weights(config, 7)
    h = torch.randn(6, 96, dtype=D64)
    qkv = P.plain_linear(h, w["h.0.attn.c_attn.weight"], w["h.0.attn.c_attn.bias"])
    q, k, v = P.plain_split_qkv(qkv, 3)
    base = P.plain_causal_attention(q, k, v)
    # zero the value columns of head 1 in the weight: exactly head 1's output vanishes
    w2 = dict(w)
    cw = w["h.0.attn.c_attn.weight"].clone()
    cb = w["h.0.attn.c_attn.bias"].clone()
    cw[:, 2 * 96 + 32: 2 * 96 + 64] = 0
    cb[2 * 96 + 32: 2 * 96 + 64] = 0
    q2, k2, v2 = P.plain_split_qkv(P.plain_linear(h, cw, cb), 3)
    out = P.plain_causal_attention(q2, k2, v2)
    assert float(out[1].abs().max()) == 0.0
    torch.testing.assert_close(out[0], base[0])
    torch.testing.assert_close(out[2], base[2])


def test_sampler_greedy_temperature_and_logprob():
    logits = torch.tensor([0.1, 2.0, -1.0, 1.9, 0.0])
    tok, lp = P.plain_sample(logits, 0.0)
    assert tok == 1
    assert abs(lp - float(torch.log_softmax(logits, -1)[1])) < 1e-6
    g = torch.Generator().manual_seed(0)
    counts = torch.zeros(5)
    n = 20000
    t = 0.7
    for _ in range(n):
        u = torch.rand(5, generator=g).clamp_min(1e-12)
        tok, lp = P.plain_sample(logits, t, gumbel=-torch.log(-torch.log(u)))
        counts[tok] += 1
    p = torch.softmax(logits / t, -1)
    sigma = torch.sqrt(p * (1 - p) / n)
    assert bool(((counts / n - p).abs() < 4 * sigma).all())
    assert abs(lp - float(torch.log_softmax(logits / t, -1)[tok])) < 1e-6


def test_stop_sequences_reference_vectors():
    # the vectors of the reference's tests/inference/test_inference_utils.py:9-88
    assert P.plain_is_stop([5, 6, 7], [[5, 6, 7]])
    assert not P.plain_is_stop([5, 6, 7], [[1, 2, 3]])
    assert P.plain_is_stop([5, 6, 7], [[6, 7]])
    assert not P.plain_is_stop([1, 2, 3], [])
    assert not P.plain_is_stop([1, 2, 3], [[]])
    assert P.plain_is_stop([8, 9, 10], [[1, 2, 3], [8, 9, 10], [4, 5, 6]])
    assert not P.plain_is_stop([28070, 5573, 323, 8254, 1667, 4227, 11, 1057, 2291, 69, 19568, 323, 40317, 743, 704], [[13]])


def test_bf16_rounding_mode_is_close_but_not_equal():
    w = P.plain_random_weights(TINY_A, 0)
    toks = torch.arange(20) % 512
    a = P.plain_logits(w, TINY_A, toks)
    b = P.plain_logits(w, TINY_A, toks, rounding=P.bf16_rounding)
    assert not torch.equal(a, b)
    assert float((a - b).abs().max()) < 0.05 * float(a.abs().max())
