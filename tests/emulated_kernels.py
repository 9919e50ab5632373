"""Plain torch statements of what each HIP kernel computes, with the kernel library's interface.

Two uses: the GPU tests compare every kernel with the function of the same name here, at sizes
other than the engine's; and the CPU tests install an instance in place of the HIP library so
that the host logic (step function, cache manager, scheduler, trace replay) runs without a GPU.
It is not part of the product: the package never imports it.
"""
from __future__ import annotations

import math
from typing import Optional

import numpy as np
import torch
import torch.nn.functional as F


def _act(name):
    return {
        "none": lambda u: u,
        "gelu": lambda u: F.gelu(u),
        "gelu_new": lambda u: F.gelu(u, approximate="tanh"),
        "relu": F.relu,
        "silu": F.silu,
        "swish": F.silu,
        "quick_gelu": lambda u: u * torch.sigmoid(1.702 * u),
        "tanh": torch.tanh,
    }[name]


# ---- Philox4x32-10 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3") in numpy ----
def philox4x32_10(c0, c1, c2, c3, k0, k1):
    c0, c1, c2, c3 = (np.asarray(c, dtype=np.uint64) for c in (c0, c1, c2, c3))
    k0 = np.uint64(k0)
    k1 = np.uint64(k1)
    mask = np.uint64(0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c0
        p1 = np.uint64(0xCD9E8D57) * c2
        n0 = ((p1 >> np.uint64(32)) ^ c1 ^ k0) & mask
        n1 = p1 & mask
        n2 = ((p0 >> np.uint64(32)) ^ c3 ^ k1) & mask
        n3 = p0 & mask
        c0, c1, c2, c3 = n0, n1, n2, n3
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c0, c1, c2, c3


def uniform_from_bits(bits: np.ndarray) -> np.ndarray:
    """(top 23 bits + 1/2) / 2^23 in float32: exact, inside (0, 1) at both ends of the range."""
    return ((bits.astype(np.uint32) >> 9).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 8388608.0)


def gumbel_from_bits(bits: np.ndarray) -> np.ndarray:
    u = uniform_from_bits(bits)
    return -np.log(-np.log(u, dtype=np.float32), dtype=np.float32)


def gumbel_noise(key0: int, key1: int, position: int, vocab: int) -> torch.Tensor:
    """The Gumbel noise the sampling kernel adds to entry v: counter (v // 4, position, 0, 0), lane v % 4."""
    groups = (vocab + 3) // 4
    g = np.arange(groups, dtype=np.uint64)
    z = np.zeros(groups, dtype=np.uint64)
    outs = philox4x32_10(g, z + np.uint64(position & 0xFFFFFFFF), z, z, key0 & 0xFFFFFFFF, key1 & 0xFFFFFFFF)
    bits = np.stack(outs, axis=1).reshape(-1)[:vocab].astype(np.uint32)
    return torch.from_numpy(gumbel_from_bits(bits))


class EmulatedKernels:
    path = "<emulated>"

    # ---- embedding
    def embed(self, tokens, positions, table, pos_table, out) -> None:
        x = table[tokens.long()].float()
        if pos_table is not None:
            x = x + pos_table[positions.long()].float()
        out.copy_(x)

    def feed_tokens(self, dst, src, rows, n) -> None:
        dst[:n] = src[:n] if rows is None else src[rows[:n].long()]

    # ---- norm
    def norm(self, x, weight, bias, eps, out, rows=None, rms=False, pending=None) -> None:
        assert pending is None, "this stand-in never leaves a product unfinished"
        src = x if rows is None else x[rows.long()]
        if rms:
            y = src / torch.sqrt((src * src).mean(-1, keepdim=True) + eps) * weight
            if bias is not None:
                y = y + bias
        else:
            y = F.layer_norm(src, (src.shape[-1],), weight, bias, eps)
        out.copy_(y.to(out.dtype))

    # ---- linear
    def linear(self, a, w, bias, out, activation="none", residual=None, may_leave_pending=False) -> None:
        y = a.float() @ w.float().t()
        if bias is not None:
            y = y + bias
        y = _act(activation)(y)
        if residual is not None:
            y = y + residual
        out.copy_(y.to(out.dtype))

    # ---- cache layout helpers:  keys [page][kvh][hd/8][ps][8], values [page][kvh][hd][ps]
    @staticmethod
    def k_view(k_pages, kvh, hd, ps):
        return k_pages.view(-1, kvh, hd // 8, ps, 8)

    @staticmethod
    def v_view(v_pages, kvh, hd, ps):
        return v_pages.view(-1, kvh, hd, ps)

    def kv_write(self, k, v, k_pages, v_pages, dest, n_kv_heads, head_dim, page_size) -> None:
        kv_ = self.k_view(k_pages, n_kv_heads, head_dim, page_size)
        vv_ = self.v_view(v_pages, n_kv_heads, head_dim, page_size)
        for t in range(k.shape[0]):
            d = int(dest[t])
            if d < 0:
                continue
            page, off = d // page_size, d % page_size
            kv_[page, :, :, off, :] = k[t].view(n_kv_heads, head_dim // 8, 8)
            vv_[page, :, :, off] = v[t].view(n_kv_heads, head_dim)

    def gather_kv(self, k_pages, v_pages, table_row, lo, hi, n_kv_heads, head_dim, page_size):
        """Keys and values of positions lo..hi-1 of one request: [kvh, n, hd] each."""
        kv_ = self.k_view(k_pages, n_kv_heads, head_dim, page_size)
        vv_ = self.v_view(v_pages, n_kv_heads, head_dim, page_size)
        ks, vs = [], []
        for p in range(lo, hi):
            page = int(table_row[p // page_size])
            assert page >= 0, "a key inside the window has no page"
            ks.append(kv_[page, :, :, p % page_size, :].reshape(n_kv_heads, head_dim))
            vs.append(vv_[page, :, :, p % page_size])
        return torch.stack(ks, 1), torch.stack(vs, 1)

    # ---- attention
    def paged_attention(self, q, out, k_pages, v_pages, meta, *, n_heads, n_kv_heads, head_dim, page_size, scale, window,
                        block_tables, k_new=None, v_new=None, dest=None, softcap=None, score_bias=None) -> bool:
        if k_new is not None:
            return False  # this stand-in never writes the cache inside attention: the caller calls kv_write
        T = q.shape[0]
        g = n_heads // n_kv_heads
        for t in range(T):
            pos = int(meta.positions[t])
            row = block_tables[int(meta.token_seq[t])]
            lo = max(0, pos - window + 1) if window else 0
            ks, vs = self.gather_kv(k_pages, v_pages, row, lo, pos + 1, n_kv_heads, head_dim, page_size)
            qt = q[t].float().view(n_heads, head_dim) * scale
            ks = ks.float().repeat_interleave(g, 0)  # [H, n, hd]
            vs = vs.float().repeat_interleave(g, 0)
            s = torch.einsum("hd,hnd->hn", qt, ks)
            if score_bias is not None:  # [heads, L]: entry min(distance, L - 1) of the head's row
                dist = (pos - torch.arange(lo, pos + 1)).clamp(max=score_bias.shape[1] - 1)
                s = s + score_bias.float().cpu()[:, dist]
            if softcap:
                s = softcap * torch.tanh(s / softcap)
            p = torch.softmax(s, -1)
            if q.dtype == torch.bfloat16:
                p = p.to(torch.bfloat16).float()
            o = torch.einsum("hn,hnd->hd", p, vs)
            out[t] = o.reshape(-1).to(out.dtype)
        return False

    # ---- sampling
    def sample(self, logits, temperatures, keys, positions, out_tokens, out_logprobs) -> None:
        for r in range(logits.shape[0]):
            lg = logits[r].float()
            temp = float(temperatures[r])
            if temp == 0.0:
                scaled = lg
                tok = int(torch.argmax(scaled))
            else:
                scaled = lg / temp
                noise = gumbel_noise(int(keys[r, 0]), int(keys[r, 1]), int(positions[r]), lg.shape[0])
                tok = int(torch.argmax(scaled + noise))
            out_tokens[r] = tok
            out_logprobs[r] = scaled[tok] - torch.logsumexp(scaled, -1)
