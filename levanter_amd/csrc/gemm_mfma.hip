// bfloat16 matrix products on the matrix cores (MFMA), 32-bit accumulation, fused epilogue:
//   y = act(a . w^T + bias) (+ residual),  a [M, K] (row stride lda), w [N, K], y [M, N] bf16 or f32.
// Two kernels:
//   tile kernel   (M > 64): 128 x 128 tile per workgroup of 4 waves, 32x32x16 MFMA, operands staged
//                 through LDS with the next tile's global loads in flight during the products;
//   skinny kernel (M <= 64): weight streaming. A workgroup owns 16 output columns; its waves split K,
//                 load their part of w straight into MFMA operand registers (16x16x32), and their
//                 partial sums are added through LDS in a fixed order (no atomics: deterministic).
// K and lda must be multiples of 8 (16-byte operand loads); any M and N.
#include "common.h"

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(16))) float f32x16;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

__device__ __forceinline__ u32x4 load16(const bf16_t* p) { return *reinterpret_cast<const u32x4*>(p); }

template <typename TO>
__device__ __forceinline__ void epilogue_store(float v, int m, int n, const float* bias, const float* residual, long ldr,
                                               TO* out, long ldo, int act) {
  if (bias) v += bias[n];
  v = lev_activate(v, act);
  if (residual) v += residual[(size_t)m * ldr + n];
  out[(size_t)m * ldo + n] = from_float<TO>(v);
}

// ------------------------------------------------------------------------------------------------
#define TM 128
#define TN 128
#define TK 32
#define LDS_STRIDE 40  // bf16 elements per LDS row: 32 + 8 of padding (80 bytes) against bank conflicts

template <typename TO>
__global__ void __launch_bounds__(256)
gemm_tile_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, const float* __restrict__ bias,
                 const float* residual, long ldr, TO* out, long ldo, int M, int N, int K, int act) {
  __shared__ __attribute__((aligned(16))) bf16_t As[2][TM * LDS_STRIDE];
  __shared__ __attribute__((aligned(16))) bf16_t Ws[2][TN * LDS_STRIDE];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * TM, n0 = blockIdx.x * TN;

  // this thread's two 16-byte chunks of each operand tile
  int lrow[2], lk[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int c = tid + 256 * i;
    lrow[i] = c >> 2;
    lk[i] = (c & 3) * 8;
  }
  u32x4 ra[2], rw[2];
  auto gload = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int k = k0 + lk[i];
      const int m = m0 + lrow[i], n = n0 + lrow[i];
      ra[i] = (m < M && k < K) ? load16(a + (size_t)m * lda + k) : u32x4{0, 0, 0, 0};
      rw[i] = (n < N && k < K) ? load16(w + (size_t)n * K + k) : u32x4{0, 0, 0, 0};
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      *reinterpret_cast<u32x4*>(&As[buf][lrow[i] * LDS_STRIDE + lk[i]]) = ra[i];
      *reinterpret_cast<u32x4*>(&Ws[buf][lrow[i] * LDS_STRIDE + lk[i]]) = rw[i];
    }
  };

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int nk = (K + TK - 1) / TK;
  gload(0);
  lstore(0);
  __syncthreads();
  const int fr = lane & 31, fk = (lane >> 5) * 8;
  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    if (kt + 1 < nk) gload((kt + 1) * TK);
#pragma unroll
    for (int ks = 0; ks < TK / 16; ++ks) {
      bf16x8 af[2], wf[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        af[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(&As[buf][(wm * 64 + i * 32 + fr) * LDS_STRIDE + ks * 16 + fk]));
        wf[i] = as_bf16x8(*reinterpret_cast<const u32x4*>(&Ws[buf][(wn * 64 + i * 32 + fr) * LDS_STRIDE + ks * 16 + fk]));
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], wf[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) lstore(buf ^ 1);
    __syncthreads();
  }

  // 32x32 accumulator: register r of lane l is row 8*(r/4) + 4*(l/32) + r%4, column l%32
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int n = n0 + wn * 64 + j * 32 + (lane & 31);
      if (n >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int m = m0 + wm * 64 + i * 32 + (r >> 2) * 8 + (lane >> 5) * 4 + (r & 3);
        if (m < M) epilogue_store<TO>(acc[i][j][r], m, n, bias, residual, ldr, out, ldo, act);
      }
    }
}

// ------------------------------------------------------------------------------------------------
// Skinny kernel. WAVES waves per workgroup; wave v takes the 32-wide k-steps v, v + WAVES, ...
// MT = number of 16-row tiles of `a` (1..4).
template <typename TO, int WAVES, int MT>
__global__ void __launch_bounds__(WAVES * 64)
gemm_skinny_kernel(const bf16_t* __restrict__ a, long lda, const bf16_t* __restrict__ w, const float* __restrict__ bias,
                   const float* residual, long ldr, TO* out, long ldo, int M, int N, int K, int act) {
  __shared__ f32x4 red[WAVES][MT][64];
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int n0 = blockIdx.x * 16;
  const int fr = lane & 15, fk = (lane >> 4) * 8;
  const int n = n0 + fr;
  const bool n_ok = n < N;
  const bf16_t* wrow = w + (size_t)(n_ok ? n : 0) * K;
  const bf16_t* arow[MT];
  bool m_ok[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    const int m = t * 16 + fr;
    m_ok[t] = m < M;
    arow[t] = a + (size_t)(m_ok[t] ? m : 0) * lda;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int nsteps = (K + 31) / 32;
  constexpr int U = MT == 1 ? 8 : 4;  // k-steps whose loads are issued together (bytes in flight per wave)
  for (int s0 = wave; s0 < nsteps; s0 += WAVES * U) {
    u32x4 wv[U];
    u32x4 av[U][MT];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int k = (s0 + u * WAVES) * 32 + fk;
      const bool k_ok = k < K;
      wv[u] = (k_ok && n_ok) ? load16(wrow + k) : u32x4{0, 0, 0, 0};
#pragma unroll
      for (int t = 0; t < MT; ++t) av[u][t] = (k_ok && m_ok[t]) ? load16(arow[t] + k) : u32x4{0, 0, 0, 0};
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < MT; ++t)
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(av[u][t]), as_bf16x8(wv[u]), acc[t], 0, 0, 0);
  }
#pragma unroll
  for (int t = 0; t < MT; ++t) red[wave][t][lane] = acc[t];
  __syncthreads();
  // 16x16 accumulator: register r of lane l is row 4*(l/16) + r, column l%16
  for (int idx = tid; idx < MT * 64; idx += WAVES * 64) {
    const int t = idx >> 6, l = idx & 63;
    f32x4 s = red[0][t][l];
#pragma unroll
    for (int v = 1; v < WAVES; ++v) {
      const f32x4 o = red[v][t][l];
      s[0] += o[0]; s[1] += o[1]; s[2] += o[2]; s[3] += o[3];
    }
    const int nn = n0 + (l & 15);
    if (nn >= N) continue;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int m = t * 16 + (l >> 4) * 4 + r;
      if (m < M) epilogue_store<TO>(s[r], m, nn, bias, residual, ldr, out, ldo, act);
    }
  }
}

template <typename TO, int WAVES>
static void launch_skinny(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr,
                          TO* out, long ldo, int M, int N, int K, int act, hipStream_t stream) {
  const int grid = (N + 15) / 16;
  const int mt = (M + 15) / 16;
#define LEV_SKINNY(MT_) \
  gemm_skinny_kernel<TO, WAVES, MT_><<<grid, WAVES * 64, 0, stream>>>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act)
  switch (mt) {
    case 1: LEV_SKINNY(1); break;
    case 2: LEV_SKINNY(2); break;
    case 3: LEV_SKINNY(3); break;
    default: LEV_SKINNY(4); break;
  }
#undef LEV_SKINNY
}

template <typename TO>
static int linear_mfma_typed(const bf16_t* a, long lda, const bf16_t* w, const float* bias, const float* residual, long ldr,
                             TO* out, long ldo, int M, int N, int K, int act, hipStream_t stream) {
  if (M <= 64) {
    if ((N + 15) / 16 >= 1024)
      launch_skinny<TO, 4>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act, stream);
    else
      launch_skinny<TO, 8>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act, stream);
  } else {
    dim3 grid((N + TN - 1) / TN, (M + TM - 1) / TM);
    if (grid.y > 65535) return lev_fail("linear: too many rows (%d) for one launch", M);
    gemm_tile_kernel<TO><<<grid, 256, 0, stream>>>(a, lda, w, bias, residual, ldr, out, ldo, M, N, K, act);
  }
  return lev_check_launch("linear_mfma");
}

extern "C" int lev_linear_mfma(const void* a, long lda, const void* w, const float* bias, const float* residual, long ldr,
                               void* out, long ldo, int M, int N, int K, int act, int out_dtype, hipStream_t stream) {
  LEV_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  LEV_REQUIRE(K % 8 == 0 && lda % 8 == 0, "linear (bfloat16): K=%d and the row stride %ld must be multiples of 8", K, lda);
  LEV_REQUIRE(((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0, "linear (bfloat16): operands must be 16-byte aligned");
  LEV_REQUIRE(lda >= K && ldo >= N, "linear: row strides lda=%ld ldo=%ld are smaller than K=%d / N=%d", lda, ldo, K, N);
  LEV_REQUIRE(!residual || (ldr >= N && out_dtype == LEV_F32), "linear: a residual needs a float32 output and a row stride >= N");
  LEV_REQUIRE(act >= LEV_ACT_NONE && act <= LEV_ACT_TANH, "linear: unknown activation %d", act);
  if (M == 0) return 0;
  if (out_dtype == LEV_F32)
    return linear_mfma_typed<float>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual, ldr, (float*)out, ldo, M, N, K,
                                    act, stream);
  if (out_dtype == LEV_BF16)
    return linear_mfma_typed<bf16_t>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual, ldr, (bf16_t*)out, ldo, M, N, K,
                                     act, stream);
  return lev_fail("linear: unknown output dtype %d", out_dtype);
}
