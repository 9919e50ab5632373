// A toy kernel that a test brings with it, outside the package: rotates the pairs (i, i + HD/2) of every head of a
// [T, heads * HD] view (row stride given) by the token's position, in place, angles and products in 32-bit.
// It includes the package's common.h for its error reporting (LEV_REQUIRE -> lev_last_error) and dtype tags.
#include "common.h"

template <typename T>
__global__ void toy_rotate_kernel(T* x, long stride, const int* __restrict__ positions, int n_heads, int HD, float base) {
  const int t = blockIdx.x, half = HD / 2;
  const float pos = (float)positions[t];
  for (int i = threadIdx.x; i < n_heads * half; i += blockDim.x) {
    const int h = i / half, j = i % half;
    const float ang = pos * powf(base, -(float)j / (float)half);
    const float c = cosf(ang), s = sinf(ang);
    T* p = x + (size_t)t * stride + (size_t)h * HD + j;
    const float a = to_float<T>(p[0]), b = to_float<T>(p[half]);
    p[0] = from_float<T>(a * c - b * s);
    p[half] = from_float<T>(b * c + a * s);
  }
}

extern "C" int toy_rotate(void* x, long stride, const int* positions, int T, int n_heads, int HD, float base, int dtype,
                          hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && n_heads > 0 && HD > 0 && HD % 2 == 0, "toy_rotate: bad sizes T=%d heads=%d head_dim=%d", T, n_heads, HD);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "toy_rotate: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    toy_rotate_kernel<float><<<T, 128, 0, stream>>>((float*)x, stride, positions, n_heads, HD, base);
  else
    toy_rotate_kernel<bf16_t><<<T, 128, 0, stream>>>((bf16_t*)x, stride, positions, n_heads, HD, base);
  return lev_check_launch("toy_rotate");
}
