// Embedding gather-add, LayerNorm / RMSNorm, the write of new keys and values into pages, sampling.
#include "common.h"
#include "sample_static.h"

// ------------------------------------------------------------------------------------------
// x[t, :] = float(table[token_t, :]) + float(pos_table[pos_t, :])        (32-bit residual stream)
// Several rows per block when rows are short; 4 elements per thread and iteration so that a row's
// loads are in flight together (a single block is bound by memory latency, not by bandwidth).
template <typename T>
__global__ void __launch_bounds__(256)
embed_kernel(const int* __restrict__ tokens, const int* __restrict__ positions, const T* __restrict__ table,
             const T* __restrict__ pos_table, float* __restrict__ out, int D) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)tokens[t] * D;
  const T* prow = pos_table ? pos_table + (size_t)positions[t] * D : nullptr;
  float* o = out + (size_t)t * D;
  if ((D & 3) == 0) {
    for (int d = threadIdx.x * 4; d < D; d += 1024) {
      float v[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) v[j] = to_float<T>(row[d + j]);
      if (prow) {
#pragma unroll
        for (int j = 0; j < 4; ++j) v[j] += to_float<T>(prow[d + j]);
      }
      *reinterpret_cast<float4*>(o + d) = make_float4(v[0], v[1], v[2], v[3]);
    }
  } else {
    for (int d = threadIdx.x; d < D; d += 256) {
      float v = to_float<T>(row[d]);
      if (prow) v += to_float<T>(prow[d]);
      o[d] = v;
    }
  }
}

extern "C" int lev_embed(const int* tokens, const int* positions, const void* table, const void* pos_table, float* out,
                         int T, int D, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && D > 0, "embed: bad sizes T=%d D=%d", T, D);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "embed: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(tokens, positions, (const float*)table, (const float*)pos_table, out, D);
  else
    embed_kernel<bf16_t><<<T, 256, 0, stream>>>(tokens, positions, (const bf16_t*)table, (const bf16_t*)pos_table, out, D);
  return lev_check_launch("embed");
}

// ------------------------------------------------------------------------------------------
// One block per output row. Statistics in 32-bit, two passes (mean, then the centred squares).
// rows != null: output row r is the norm of input row rows[r] (the wanted rows before the head).
// Rows of up to NT * 4 * NV floats are read once, as float4, into registers: every load of the row is in
// flight at the same time. Longer rows (or a width that is no multiple of 4) take the looping kernel.
template <typename TO>
__device__ __forceinline__ void store4(TO* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<float4*>(p) = make_float4(a, b, c, d);
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
  uint2 v;
  v.x = float2_to_bf16x2(a, b);
  v.y = float2_to_bf16x2(c, d);
  *reinterpret_cast<uint2*>(p) = v;
}

// partial != null: the row is first brought up to date. A matrix product that split its sum into S ranges has left
// them in partial [S][M][D] instead of adding them to x (its residual); here x[row] += (partial[0] + .. + partial[S-1]
// + lin_bias), in that order, is stored back and normalised in the same pass: one kernel where a reduction kernel and a
// norm kernel would each read and write the row. With a selection of rows (rows != null) nothing is stored back: the rows
// that are left out stay unfinished anyway, so x as a whole is of no use afterwards, and a row that the selection names
// twice would otherwise be read by one workgroup while another has already stored its new value.
template <typename TO, int NT, int NV>
__global__ void __launch_bounds__(NT)
norm_reg_kernel(float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b, TO* __restrict__ out,
                const int* __restrict__ rows, int D, float eps, int rms, const float* __restrict__ partial, int S,
                size_t partial_stride, const float* __restrict__ lin_bias) {
  __shared__ float red[NT / 64];
  const int r = blockIdx.x;
  const size_t row = (size_t)(rows ? rows[r] : r);
  float* xr = x + row * D;
  // the row, and scale and shift with it: their latency passes during the two reductions
  float4 v[NV], wv[NV], bv[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int d = (threadIdx.x + i * NT) * 4;
    const bool ok = d < D;
    v[i] = ok ? *reinterpret_cast<const float4*>(xr + d) : make_float4(0.f, 0.f, 0.f, 0.f);
    wv[i] = ok ? *reinterpret_cast<const float4*>(w + d) : make_float4(0.f, 0.f, 0.f, 0.f);
    bv[i] = ok && b ? *reinterpret_cast<const float4*>(b + d) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if (partial) {
    const float* pr = partial + row * D;
#pragma unroll
    for (int i = 0; i < NV; ++i) {
      const int d = (threadIdx.x + i * NT) * 4;
      if (d < D) {
        float4 t = make_float4(0.f, 0.f, 0.f, 0.f);
        int s = 0;
        for (; s + 4 <= S; s += 4) {  // four ranges requested at once, added in their order
          float4 p[4];
#pragma unroll
          for (int j = 0; j < 4; ++j) p[j] = *reinterpret_cast<const float4*>(pr + (size_t)(s + j) * partial_stride + d);
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            t.x += p[j].x; t.y += p[j].y; t.z += p[j].z; t.w += p[j].w;
          }
        }
        for (; s < S; ++s) {
          const float4 p = *reinterpret_cast<const float4*>(pr + (size_t)s * partial_stride + d);
          t.x += p.x; t.y += p.y; t.z += p.z; t.w += p.w;
        }
        if (lin_bias) {
          const float4 lb = *reinterpret_cast<const float4*>(lin_bias + d);
          t.x += lb.x; t.y += lb.y; t.z += lb.z; t.w += lb.w;
        }
        v[i].x = t.x + v[i].x; v[i].y = t.y + v[i].y; v[i].z = t.z + v[i].z; v[i].w = t.w + v[i].w;
        if (!rows) *reinterpret_cast<float4*>(xr + d) = v[i];
      }
    }
  }
  float mean = 0.f;
  if (!rms) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < NV; ++i) s += (v[i].x + v[i].y) + (v[i].z + v[i].w);
    mean = block_sum<NT>(s, red) / (float)D;
  }
  float s2 = 0.f;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int d = (threadIdx.x + i * NT) * 4;
    if (d < D) {
      const float c0 = v[i].x - mean, c1 = v[i].y - mean, c2 = v[i].z - mean, c3 = v[i].w - mean;
      s2 += (c0 * c0 + c1 * c1) + (c2 * c2 + c3 * c3);
    }
  }
  const float var = block_sum<NT>(s2, red) / (float)D;
  const float rstd = 1.0f / sqrtf(var + eps);
  TO* o = out + (size_t)r * D;
#pragma unroll
  for (int i = 0; i < NV; ++i) {
    const int d = (threadIdx.x + i * NT) * 4;
    if (d < D)
      store4<TO>(o + d, (v[i].x - mean) * rstd * wv[i].x + bv[i].x, (v[i].y - mean) * rstd * wv[i].y + bv[i].y,
                 (v[i].z - mean) * rstd * wv[i].z + bv[i].z, (v[i].w - mean) * rstd * wv[i].w + bv[i].w);
  }
}

template <typename TO, int NT>
__global__ void norm_kernel(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b,
                            TO* __restrict__ out, const int* __restrict__ rows, int D, float eps, int rms) {
  __shared__ float red[NT / 64];
  const int r = blockIdx.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * D;
  float mean = 0.f;
  if (!rms) {
    float s = 0.f;
    for (int d = threadIdx.x; d < D; d += NT) s += xr[d];
    mean = block_sum<NT>(s, red) / (float)D;
  }
  float s2 = 0.f;
  for (int d = threadIdx.x; d < D; d += NT) {
    float c = xr[d] - mean;
    s2 += c * c;
  }
  const float var = block_sum<NT>(s2, red) / (float)D;
  const float rstd = 1.0f / sqrtf(var + eps);
  TO* o = out + (size_t)r * D;
  for (int d = threadIdx.x; d < D; d += NT) {
    float y = (xr[d] - mean) * rstd * w[d];
    if (b) y += b[d];
    o[d] = from_float<TO>(y);
  }
}

// Returns false if a pending sum (partial != null) cannot be folded in at this width and alignment: the caller then
// runs the reduction by itself first.
template <typename TO>
static bool launch_norm(float* x, const float* w, const float* b, TO* out, const int* rows, int n_rows, int D, float eps,
                        int rms, const float* partial, int S, size_t partial_stride, const float* lin_bias, hipStream_t stream) {
  // rows in registers as vectors of 4: needs D % 4 == 0 and 16-byte aligned pointers
  const bool vec = (D & 3) == 0 && (((uintptr_t)x | (uintptr_t)w | (uintptr_t)b | (uintptr_t)out | (uintptr_t)partial |
                                     (uintptr_t)lin_bias) & 15) == 0 && (partial_stride & 3) == 0;
  // With ranges to add, a row is S + 1 times as many bytes and there are few rows (a decode batch): 1,024 threads a row,
  // every load of the row and its ranges in flight at once (with 256 threads 64 workgroups took longer over 17 MB of
  // ranges than the reduction kernel and the norm kernel together).
  if (partial && vec && D <= 1024 * 4)
    norm_reg_kernel<TO, 1024, 1><<<n_rows, 1024, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  else if (partial && vec && D <= 1024 * 4 * 2)
    norm_reg_kernel<TO, 1024, 2><<<n_rows, 1024, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  else if (vec && D <= 256 * 4 * 2)
    norm_reg_kernel<TO, 256, 2><<<n_rows, 256, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  // 512 threads from 2,048 columns on: a row's loads are fewer per thread and the kernel is latency from end to end
  // (8 rows of 4,096: 2.8 us against 3.1 with 256 threads, 3.1 with 1,024; of 6,144: 3.3 against 3.8)
  else if (vec && D <= 512 * 4 * 2)
    norm_reg_kernel<TO, 512, 2><<<n_rows, 512, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  else if (vec && D <= 512 * 4 * 3)
    norm_reg_kernel<TO, 512, 3><<<n_rows, 512, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  else if (vec && D <= 256 * 4 * 8)
    norm_reg_kernel<TO, 256, 8><<<n_rows, 256, 0, stream>>>(x, w, b, out, rows, D, eps, rms, partial, S, partial_stride, lin_bias);
  else if (partial)
    return false;
  else
    norm_kernel<TO, 256><<<n_rows, 256, 0, stream>>>(x, w, b, out, rows, D, eps, rms);
  return true;
}

extern "C" int lev_norm(const float* x, const float* w, const float* b, void* out, const int* rows, int n_rows, int D,
                        float eps, int rms, int out_dtype, hipStream_t stream) {
  LEV_REQUIRE(n_rows >= 0 && D > 0, "norm: bad sizes rows=%d D=%d", n_rows, D);
  LEV_REQUIRE(out_dtype == LEV_F32 || out_dtype == LEV_BF16, "norm: unknown output dtype %d", out_dtype);
  LEV_REQUIRE(eps > 0.f, "norm: eps must be positive");
  if (n_rows == 0) return 0;
  if (out_dtype == LEV_F32)
    launch_norm<float>(const_cast<float*>(x), w, b, (float*)out, rows, n_rows, D, eps, rms, nullptr, 0, 0, nullptr, stream);
  else
    launch_norm<bf16_t>(const_cast<float*>(x), w, b, (bf16_t*)out, rows, n_rows, D, eps, rms, nullptr, 0, 0, nullptr, stream);
  return lev_check_launch("norm");
}

// The norm of rows that a matrix product has not finished yet: x [M][D] + partial[0] + .. + partial[S-1] + lin_bias, then the
// norm as in lev_norm. rows == null: all M rows, and the sums are stored back into x, which is then finished. rows given:
// only those rows are summed and normalised and x is left as it was (unfinished; a row may be named more than once).
// Returns 1, with nothing launched, if this width or alignment has no such kernel.
extern "C" int lev_norm_pending(float* x, const float* partial, int S, const float* lin_bias, const float* w, const float* b,
                                void* out, const int* rows, int n_rows, int M, int D, float eps, int rms, int out_dtype,
                                hipStream_t stream) {
  LEV_REQUIRE(n_rows >= 0 && D > 0 && M > 0 && S >= 1 && partial, "norm: bad sizes rows=%d D=%d M=%d ranges=%d", n_rows, D, M, S);
  LEV_REQUIRE(out_dtype == LEV_F32 || out_dtype == LEV_BF16, "norm: unknown output dtype %d", out_dtype);
  LEV_REQUIRE(eps > 0.f, "norm: eps must be positive");
  if (n_rows == 0) return 0;
  const size_t stride = (size_t)M * D;
  const bool ok = out_dtype == LEV_F32
                      ? launch_norm<float>(x, w, b, (float*)out, rows, n_rows, D, eps, rms, partial, S, stride, lin_bias, stream)
                      : launch_norm<bf16_t>(x, w, b, (bf16_t*)out, rows, n_rows, D, eps, rms, partial, S, stride, lin_bias, stream);
  if (!ok) return 1;
  return lev_check_launch("norm");
}

// ------------------------------------------------------------------------------------------
// New keys and values into their pages. Page layouts (elements):
//   keys   [page][kv_head][head_dim/8][page_size][8]
//   values [page][kv_head][head_dim][page_size]
// dest[t] = page * page_size + offset in page; a negative dest drops the token.
// A workgroup takes KVW_TOKENS consecutive tokens of the batch and one kv head. A key chunk of 8 elements is
// contiguous on both sides: 16-byte (bf16) copies. Values are transposed through LDS: where 8 tokens in a row go
// to 8 consecutive, aligned slots of one page (a prompt portion does, except at its ragged ends), a thread writes
// its head-dim row for all 8 at once; other tokens are written element by element.
#define KVW_TOKENS 16

template <typename T>
__device__ __forceinline__ void copy8(T* dst, const T* src) {  // 8 elements, both 16-byte aligned
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
#pragma unroll
  for (int i = 0; i < (int)(8 * sizeof(T) / 16); ++i)
    reinterpret_cast<u32x4*>(dst)[i] = reinterpret_cast<const u32x4*>(src)[i];
}

template <typename T>
__global__ void kv_write_kernel(const T* __restrict__ k, const T* __restrict__ v, long k_stride, long v_stride,
                                T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ dest, int n_tokens,
                                int KVH, int HD, int PS, int vec_ok) {
  extern __shared__ __attribute__((aligned(16))) unsigned char kvw_smem[];
  int* dst_s = reinterpret_cast<int*>(kvw_smem);                       // [KVW_TOKENS]
  T* vt = reinterpret_cast<T*>(kvw_smem + KVW_TOKENS * sizeof(int));   // [KVW_TOKENS][HD + 8]
  const int ldv = HD + 8;
  const int t0 = blockIdx.x * KVW_TOKENS;
  const int h = blockIdx.y;
  const int tid = threadIdx.x;
  if (tid < KVW_TOKENS) dst_s[tid] = t0 + tid < n_tokens ? dest[t0 + tid] : -1;
  const int chunks = HD / 8;
  // keys: one chunk of one token per thread and turn; values into LDS on the way
  for (int idx = tid; idx < KVW_TOKENS * chunks; idx += blockDim.x) {
    const int i = idx / chunks, c = idx % chunks;
    const int t = t0 + i;
    if (t >= n_tokens) continue;
    const int dst = dest[t];
    if (dst < 0) continue;
    const T* kr = k + (size_t)t * k_stride + (size_t)h * HD + c * 8;
    const T* vr = v + (size_t)t * v_stride + (size_t)h * HD + c * 8;
    const int page = dst / PS, off = dst % PS;
    T* kd = k_pages + ((size_t)page * KVH + h) * (size_t)HD * PS + ((size_t)c * PS + off) * 8;
    if (vec_ok) {
      copy8<T>(kd, kr);
      copy8<T>(vt + i * ldv + c * 8, vr);
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        kd[e] = kr[e];
        vt[i * ldv + c * 8 + e] = vr[e];
      }
    }
  }
  __syncthreads();
  for (int d = tid; d < HD; d += blockDim.x) {
    int i = 0;
    while (i < KVW_TOKENS) {
      const int dst = dst_s[i];
      if (dst < 0) {
        ++i;
        continue;
      }
      const int page = dst / PS, off = dst % PS;
      T* vd = v_pages + ((size_t)page * KVH + h) * (size_t)HD * PS + (size_t)d * PS + off;
      bool run = vec_ok && (off % 8 == 0) && i + 8 <= KVW_TOKENS;
      if (run) {
#pragma unroll
        for (int j = 1; j < 8; ++j) run = run && dst_s[i + j] == dst + j;
      }
      if (run) {
        __attribute__((aligned(16))) T row[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) row[j] = vt[(i + j) * ldv + d];
        copy8<T>(vd, row);
        i += 8;
      } else {
        *vd = vt[i * ldv + d];
        ++i;
      }
    }
  }
}

extern "C" int lev_kv_write(const void* k, const void* v, long k_stride, long v_stride, void* k_pages, void* v_pages,
                            const int* dest, int T, int KVH, int HD, int PS, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && KVH > 0, "kv_write: bad sizes T=%d kv_heads=%d", T, KVH);
  LEV_REQUIRE(HD > 0 && HD % 8 == 0, "kv_write: head_dim=%d must be a multiple of 8", HD);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "kv_write: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(KVH <= 65535, "kv_write: too many kv heads (%d)", KVH);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "kv_write: unknown dtype %d", dtype);
  if (T == 0) return 0;
  const size_t esize = dtype == LEV_F32 ? 4 : 2;
  const size_t lds = KVW_TOKENS * sizeof(int) + (size_t)KVW_TOKENS * (HD + 8) * esize;
  LEV_REQUIRE(lds <= 64 * 1024, "kv_write: head_dim=%d is too large", HD);
  // 16-byte copies of the source rows need aligned rows (the pages always are: page_size and head_dim are multiples of 8)
  const int vec_ok = ((uintptr_t)k % 16 == 0) && ((uintptr_t)v % 16 == 0) && (k_stride * esize % 16 == 0) && (v_stride * esize % 16 == 0) &&
                     ((uintptr_t)k_pages % 16 == 0) && ((uintptr_t)v_pages % 16 == 0);
  dim3 grid((T + KVW_TOKENS - 1) / KVW_TOKENS, KVH);
  const int nt = HD <= 64 ? 64 : (HD <= 128 ? 128 : 256);
  if (dtype == LEV_F32)
    kv_write_kernel<float><<<grid, nt, lds, stream>>>((const float*)k, (const float*)v, k_stride, v_stride, (float*)k_pages,
                                                      (float*)v_pages, dest, T, KVH, HD, PS, vec_ok);
  else
    kv_write_kernel<bf16_t><<<grid, nt, lds, stream>>>((const bf16_t*)k, (const bf16_t*)v, k_stride, v_stride,
                                                       (bf16_t*)k_pages, (bf16_t*)v_pages, dest, T, KVH, HD, PS, vec_ok);
  return lev_check_launch("kv_write");
}

// ------------------------------------------------------------------------------------------
// Sampling. One block per row of 32-bit logits.
//   temperature == 0: token = argmax(logits) (ties: the lowest index), logprob from the raw logits;
//   otherwise: token = argmax(logits / T + Gumbel noise), logprob = (logits/T)[token] - logsumexp(logits/T).
// The noise of vocabulary entry v comes from Philox4x32-10 with the row's 64-bit key and the counter
// (v / 4, position, 0, 0), lane v % 4: it depends on (key, position, v) and on nothing else.
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3, uint32_t k0, uint32_t k1,
                                              uint32_t out[4]) {
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint64_t p0 = (uint64_t)0xD2511F53u * c0;
    const uint64_t p1 = (uint64_t)0xCD9E8D57u * c2;
    const uint32_t n0 = (uint32_t)(p1 >> 32) ^ c1 ^ k0;
    const uint32_t n1 = (uint32_t)p1;
    const uint32_t n2 = (uint32_t)(p0 >> 32) ^ c3 ^ k1;
    const uint32_t n3 = (uint32_t)p0;
    c0 = n0; c1 = n1; c2 = n2; c3 = n3;
    k0 += 0x9E3779B9u;
    k1 += 0xBB67AE85u;
  }
  out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

// u = (top 23 bits + 1/2) / 2^23: every value is a float32 exactly (24 significant bits at most), the smallest is 2^-24 and the
// largest 1 - 2^-24, so both logarithms are finite. (With 24 bits the largest sum would round up to 1 and the noise to +inf.)
__device__ __forceinline__ float gumbel_from_bits(uint32_t bits) {
  const float u = ((float)(bits >> 9) + 0.5f) * (1.0f / 8388608.0f);
  return -logf(-logf(u));
}

struct ArgMax {
  float v;
  int i;
};
__device__ __forceinline__ ArgMax better(ArgMax a, ArgMax b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

// Stage 1: block (row, part) scans its part of the vocabulary: best candidate, maximum of the scaled
// logits and the sum of exp(scaled - that maximum). Stage 2: one wave per row merges the parts in order.
#define SAMPLE_PARTS 64

template <int NT>
__global__ void __launch_bounds__(NT)
sample_part_kernel(const float* __restrict__ logits, long row_stride, const float* __restrict__ temperature,
                   const uint32_t* __restrict__ keys, const int* __restrict__ positions, float* __restrict__ part, int V) {
  __shared__ float red[NT / 64];
  __shared__ float sv[NT / 64];
  __shared__ int si[NT / 64];
  const int r = blockIdx.x, b = blockIdx.y;
  const float* lg = logits + (size_t)r * row_stride;
  const float temp = temperature[r];
  const bool greedy = (temp == 0.0f);
  const float safe_t = greedy ? 1.0f : temp;
  const uint32_t k0 = keys[2 * r], k1 = keys[2 * r + 1];
  const uint32_t pos = (uint32_t)positions[r];
  const int groups = (V + 3) / 4;
  const int per = (groups + SAMPLE_PARTS - 1) / SAMPLE_PARTS;
  const int g_begin = b * per, g_end = min(groups, g_begin + per);

  ArgMax best = {-INFINITY, 0x7fffffff};
  float mx = -INFINITY;
  for (int g = g_begin + threadIdx.x; g < g_end; g += NT) {
    uint32_t rnd[4] = {0, 0, 0, 0};
    if (!greedy) philox4x32_10((uint32_t)g, pos, 0u, 0u, k0, k1, rnd);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int v = g * 4 + j;
      if (v < V) {
        const float s = lg[v] / safe_t;
        mx = fmaxf(mx, s);
        const float c = greedy ? s : s + gumbel_from_bits(rnd[j]);
        best = better(best, ArgMax{c, v});
      }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax other = {__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
    best = better(best, other);
  }
  if ((threadIdx.x & 63) == 0) {
    sv[threadIdx.x >> 6] = best.v;
    si[threadIdx.x >> 6] = best.i;
  }
  mx = block_max<NT>(mx, red);  // syncs: sv / si are visible afterwards
  ArgMax top = {sv[0], si[0]};
#pragma unroll
  for (int i = 1; i < NT / 64; ++i) top = better(top, ArgMax{sv[i], si[i]});
  float se = 0.f;
  if (mx != -INFINITY)
    for (int g = g_begin + threadIdx.x; g < g_end; g += NT)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int v = g * 4 + j;
        if (v < V) se += expf(lg[v] / safe_t - mx);
      }
  se = block_sum<NT>(se, red);
  if (threadIdx.x == 0) {
    float* p = part + ((size_t)r * SAMPLE_PARTS + b) * 4;
    p[0] = top.v;
    p[1] = __int_as_float(top.i);
    p[2] = mx;
    p[3] = se;
  }
}

__global__ void __launch_bounds__(64)
sample_merge_kernel(const float* __restrict__ logits, long row_stride, const float* __restrict__ temperature,
                    const float* __restrict__ part, int* __restrict__ tokens, float* __restrict__ logprobs, int V) {
  const int r = blockIdx.x, lane = threadIdx.x;
  const float* p = part + ((size_t)r * SAMPLE_PARTS + lane) * 4;
  ArgMax best = {p[0], __float_as_int(p[1])};
  const float mxb = p[2], seb = p[3];
  const float mx = wave_max(mxb);
  const float se = wave_sum(mxb == -INFINITY ? 0.f : seb * expf(mxb - mx));
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    ArgMax other = {__shfl_xor(best.v, o, 64), __shfl_xor(best.i, o, 64)};
    best = better(best, other);
  }
  if (lane == 0) {
    const float temp = temperature[r];
    const float safe_t = temp == 0.0f ? 1.0f : temp;
    const int tok = best.i < V ? best.i : 0;
    tokens[r] = tok;
    logprobs[r] = logits[(size_t)r * row_stride + tok] / safe_t - mx - logf(se);
  }
}

extern "C" long lev_sample_workspace(int R) { return (long)R * SAMPLE_PARTS * 4 * (long)sizeof(float); }

extern "C" int lev_sample(const float* logits, long row_stride, const float* temperature, const uint32_t* keys,
                          const int* positions, int* tokens, float* logprobs, float* workspace, int R, int V,
                          hipStream_t stream) {
  LEV_REQUIRE(R >= 0 && V > 0, "sample: bad sizes rows=%d vocab=%d", R, V);
  LEV_REQUIRE(row_stride >= V, "sample: row stride %ld is smaller than the vocabulary %d", row_stride, V);
  LEV_REQUIRE(R <= 65535 * 16, "sample: too many rows (%d)", R);
  if (R == 0) return 0;
  LEV_REQUIRE(workspace != nullptr, "sample: a workspace of lev_sample_workspace(rows) bytes is needed");
  static_assert(SAMPLE_PARTS == 64, "the merge kernel reads one part per lane");
  sample_part_kernel<256><<<dim3(R, SAMPLE_PARTS), 256, 0, stream>>>(logits, row_stride, temperature, keys, positions, workspace, V);
  if (int rc = lev_check_launch("sample")) return rc;
  sample_merge_kernel<<<R, 64, 0, stream>>>(logits, row_stride, temperature, workspace, tokens, logprobs, V);
  return lev_check_launch("sample merge");
}

// ------------------------------------------------------------------------------------------
// Token ids of a step that were sampled by the step before and are still on the device: dst[i] = src[rows ? rows[i] : i].
__global__ void feed_tokens_kernel(int* __restrict__ dst, const int* __restrict__ src, const int* __restrict__ rows, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] = src[rows ? rows[i] : i];
}

extern "C" int lev_feed_tokens(int* dst, const int* src, const int* rows, int n, hipStream_t stream) {
  LEV_REQUIRE(n >= 0 && (n == 0 || (dst && src)), "feed_tokens: bad arguments (n=%d)", n);
  if (n == 0) return 0;
  feed_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(dst, src, rows, n);
  return lev_check_launch("feed_tokens");
}

// ---- the same sampling from a scratch array of the library's own (see sample_static.h) -----------------------
// In host code `sample_scratch` is only a stand-in for the symbol: the address a kernel can use comes from
// hipGetSymbolAddress, once per device, and is kept in g_sample_scratch[device].
#define LEV_MAX_DEVICES 64
static __device__ __align__(256) float sample_scratch[(size_t)LEV_SAMPLE_STATIC_MAX_ROWS * SAMPLE_PARTS * 4];
static float* g_sample_scratch[LEV_MAX_DEVICES];  // written once per device with one value: racing initialisers agree

static int sample_scratch_ptr(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return lev_fail("sample_static: hipGetDevice failed: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= LEV_MAX_DEVICES) return lev_fail("sample_static: device %d is beyond the %d this library keeps scratch for", dev, LEV_MAX_DEVICES);
  float* p = __atomic_load_n(&g_sample_scratch[dev], __ATOMIC_ACQUIRE);
  if (!p) {
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(sample_scratch));
    if (e != hipSuccess || !p) return lev_fail("sample_static: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
    __atomic_store_n(&g_sample_scratch[dev], p, __ATOMIC_RELEASE);
  }
  *out = p;
  return 0;
}

extern "C" int lev_sample_static_init() {
  float* p = nullptr;
  return sample_scratch_ptr(&p);
}

extern "C" int lev_sample_static_max_rows() { return LEV_SAMPLE_STATIC_MAX_ROWS; }

extern "C" int lev_sample_static(const float* logits, long row_stride, const float* temperature, const uint32_t* keys,
                                 const int* positions, int* tokens, float* logprobs, int R, int V, hipStream_t stream) {
  LEV_REQUIRE(R <= LEV_SAMPLE_STATIC_MAX_ROWS, "sample_static: %d rows are more than the %d its scratch array holds; use lev_sample with a workspace",
              R, LEV_SAMPLE_STATIC_MAX_ROWS);
  float* scratch = nullptr;
  if (int rc = sample_scratch_ptr(&scratch)) return rc;
  return lev_sample(logits, row_stride, temperature, keys, positions, tokens, logprobs, scratch, R, V, stream);
}
