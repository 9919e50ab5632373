// Attention of a ragged batch of query tokens over the paged cache, with plain 32-bit arithmetic:
// the attention of the true 32-bit path, and a size-agnostic one for bfloat16 caches.
// One wave per (query token, head). Keys are visited 64 at a time with an online softmax.
//   q     [T][H*HD] (row stride q_stride), out likewise
//   keys  [page][kv_head][HD/8][PS][8], values [page][kv_head][HD][PS]
//   positions[t]: absolute position of query t; it sees keys at positions p with
//                 max(0, pos - window + 1) <= p <= pos   (window 0: all)
//   token_seq[t]: row of block_tables (page ids of that request, -1 where none). A key whose block has no page
//                 is treated as masked and never loaded (a padding token of a replayed step may name a block that
//                 its request has given back); a query with no key at all gives zeros.
#include "common.h"

#define AS_MAX_HD 512

template <typename T>
__global__ void __launch_bounds__(64)
attention_simple_kernel(const T* __restrict__ q, long q_stride, T* __restrict__ out, long o_stride,
                        const T* __restrict__ k_pages, const T* __restrict__ v_pages, const int* __restrict__ positions,
                        const int* __restrict__ token_seq, const int* __restrict__ block_tables, int bt_stride, int H,
                        int KVH, int HD, int PS, float scale, int window, float softcap, const float* __restrict__ score_bias,
                        int bias_len) {
  __shared__ float qs[AS_MAX_HD];
  __shared__ float ps[64];
  __shared__ int pg[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (H / KVH);
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * bt_stride;
  for (int d = lane; d < HD; d += 64) qs[d] = to_float<T>(q[(size_t)t * q_stride + (size_t)h * HD + d]) * scale;
  const int first = window > 0 ? max(0, pos - window + 1) : 0;
  constexpr int ND = AS_MAX_HD / 64;
  float acc[ND];
#pragma unroll
  for (int i = 0; i < ND; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  __syncthreads();
  const size_t head_elems = (size_t)HD * PS;
  for (int c0 = (first / 64) * 64; c0 <= pos; c0 += 64) {
    const int kp = c0 + lane;
    bool live = kp >= first && kp <= pos;
    float s = -INFINITY;
    int page = -1;
    if (live) page = bt[kp / PS];
    live = live && page >= 0;
    if (live) {
      const int off = kp % PS;
      const T* kb = k_pages + ((size_t)page * KVH + kvh) * head_elems;
      float dot = 0.f;
      for (int d = 0; d < HD; ++d) dot = fmaf(qs[d], to_float<T>(kb[((size_t)(d >> 3) * PS + off) * 8 + (d & 7)]), dot);
      // between the scaling and the mask a model may add a term per (head, distance) and cap the score softly
      // (src/levanter/layers/attention.py:361-367); both are off unless asked for
      if (score_bias) dot += score_bias[(size_t)h * bias_len + min(pos - kp, bias_len - 1)];
      if (softcap > 0.f) dot = softcap * tanhf(dot / softcap);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = live ? expf(s - m_new) : 0.f;  // no live key so far: m_new = -inf, p = 0
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    pg[lane] = page;
    __syncthreads();
    const int n_live = min(64, pos - c0 + 1);
#pragma unroll
    for (int i = 0; i < ND; ++i) {
      const int d = lane + 64 * i;
      if (d < HD) {
        float a = acc[i] * corr;
        for (int j = 0; j < n_live; ++j) {
          const int pj = pg[j];
          if (pj >= 0) {
            const T* vb = v_pages + ((size_t)pj * KVH + kvh) * head_elems;
            a = fmaf(ps[j], to_float<T>(vb[(size_t)d * PS + (c0 + j) % PS]), a);
          }
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int i = 0; i < ND; ++i) {
    const int d = lane + 64 * i;
    if (d < HD) out[(size_t)t * o_stride + (size_t)h * HD + d] = from_float<T>(acc[i] * inv);
  }
}

extern "C" int lev_attention_simple(const void* q, long q_stride, void* out, long o_stride, const void* k_pages,
                                    const void* v_pages, const int* positions, const int* token_seq, const int* block_tables,
                                    int bt_stride, int T, int H, int KVH, int HD, int PS, float scale, int window, int dtype,
                                    float softcap, const float* score_bias, int bias_len, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H > 0 && KVH > 0 && H % KVH == 0, "attention: bad head counts heads=%d kv_heads=%d", H, KVH);
  LEV_REQUIRE(HD > 0 && HD % 8 == 0 && HD <= AS_MAX_HD, "attention: head_dim=%d must be a multiple of 8 and at most %d", HD,
              AS_MAX_HD);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "attention: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(H <= 65535, "attention: too many heads (%d)", H);
  LEV_REQUIRE(window >= 0, "attention: window=%d must not be negative", window);
  LEV_REQUIRE(softcap >= 0.f && (!score_bias || bias_len >= 1), "attention: soft cap %g must not be negative and a bias table needs entries (%d)",
              (double)softcap, bias_len);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "attention: unknown dtype %d", dtype);
  if (T == 0) return 0;
  dim3 grid(T, H);
  if (dtype == LEV_F32)
    attention_simple_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_stride, (float*)out, o_stride,
                                                           (const float*)k_pages, (const float*)v_pages, positions, token_seq,
                                                           block_tables, bt_stride, H, KVH, HD, PS, scale, window, softcap, score_bias, bias_len);
  else
    attention_simple_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_stride, (bf16_t*)out, o_stride,
                                                            (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions,
                                                            token_seq, block_tables, bt_stride, H, KVH, HD, PS, scale, window, softcap, score_bias,
                                                            bias_len);
  return lev_check_launch("attention_simple");
}
