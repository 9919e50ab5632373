// y = act(a . w^T + bias) + residual with plain fused multiply-adds in 32-bit: the matrix product
// of the true 32-bit path (no matrix-core instruction, no reduced-precision mode) and a slow but
// size-agnostic product for bfloat16 inputs.  a [M, K] (row stride lda), w [N, K], y [M, N].
#include "common.h"

#define GS_TILE 64
#define GS_BK 16

template <typename TI, typename TO>
__global__ void __launch_bounds__(256)
gemm_simple_kernel(const TI* __restrict__ a, long lda, const TI* __restrict__ w, const float* __restrict__ bias,
                   const float* residual, long ldr, TO* out, long ldo, int M, int N, int K, int act) {
  __shared__ float As[GS_BK][GS_TILE + 4];
  __shared__ float Ws[GS_BK][GS_TILE + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GS_TILE, n0 = blockIdx.x * GS_TILE;
  const int lrow = tid >> 2, lk = (tid & 3) * 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GS_BK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + lk + j;
      const int m = m0 + lrow, n = n0 + lrow;
      As[lk + j][lrow] = (m < M && k < K) ? to_float<TI>(a[(size_t)m * lda + k]) : 0.f;
      Ws[lk + j][lrow] = (n < N && k < K) ? to_float<TI>(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < GS_BK; ++k) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) av[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) wv[j] = Ws[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n >= N) continue;
      float v = acc[i][j];
      if (bias) v += bias[n];
      v = lev_activate(v, act);
      if (residual) v += residual[(size_t)m * ldr + n];
      out[(size_t)m * ldo + n] = from_float<TO>(v);
    }
  }
}

extern "C" int lev_linear_simple(const void* a, long lda, const void* w, const float* bias, const float* residual, long ldr,
                                 void* out, long ldo, int M, int N, int K, int act, int in_dtype, int out_dtype,
                                 hipStream_t stream) {
  LEV_REQUIRE(M >= 0 && N > 0 && K > 0, "linear: bad sizes M=%d N=%d K=%d", M, N, K);
  LEV_REQUIRE(lda >= K && ldo >= N, "linear: row strides lda=%ld ldo=%ld are smaller than K=%d / N=%d", lda, ldo, K, N);
  LEV_REQUIRE(!residual || ldr >= N, "linear: residual row stride %ld is smaller than N=%d", ldr, N);
  LEV_REQUIRE(act >= LEV_ACT_NONE && act <= LEV_ACT_TANH, "linear: unknown activation %d", act);
  if (M == 0) return 0;
  dim3 grid((N + GS_TILE - 1) / GS_TILE, (M + GS_TILE - 1) / GS_TILE);
  LEV_REQUIRE(grid.y <= 65535, "linear: too many rows (%d) for one launch", M);
  if (in_dtype == LEV_F32 && out_dtype == LEV_F32)
    gemm_simple_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)a, lda, (const float*)w, bias, residual, ldr,
                                                               (float*)out, ldo, M, N, K, act);
  else if (in_dtype == LEV_BF16 && out_dtype == LEV_F32)
    gemm_simple_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual,
                                                                ldr, (float*)out, ldo, M, N, K, act);
  else if (in_dtype == LEV_BF16 && out_dtype == LEV_BF16)
    gemm_simple_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, lda, (const bf16_t*)w, bias, residual,
                                                                 ldr, (bf16_t*)out, ldo, M, N, K, act);
  else
    return lev_fail("linear: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
  return lev_check_launch("linear_simple");
}
