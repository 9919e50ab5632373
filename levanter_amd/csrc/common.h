// Shared helpers of the HIP sources: error reporting, dtype tags, reductions, bf16 conversion.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

enum LevDtype { LEV_F32 = 0, LEV_BF16 = 1 };
enum LevAct { LEV_ACT_NONE = 0, LEV_ACT_GELU_TANH = 1, LEV_ACT_GELU_ERF = 2, LEV_ACT_RELU = 3, LEV_ACT_SILU = 4,
              LEV_ACT_QUICK_GELU = 5, LEV_ACT_TANH = 6 };

// ---- errors: every entry point returns 0 or a negative code and leaves a message here
extern "C" const char* lev_last_error();
int lev_fail(const char* fmt, ...);
int lev_check_launch(const char* what);

#define LEV_REQUIRE(cond, ...)            \
  do {                                    \
    if (!(cond)) return lev_fail(__VA_ARGS__); \
  } while (0)

// ---- bf16 as raw 16 bits -----------------------------------------------------------------
typedef uint16_t bf16_t;

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even with the hardware conversion of gfx950 (v_cvt_pk_bf16_f32); NaN stays NaN
__device__ __forceinline__ bf16_t float_to_bf16(float f) {
  union { __bf16 b; bf16_t u; } c;
  c.b = (__bf16)f;
  return c.u;
}
// two values at once: lo in the low half
__device__ __forceinline__ uint32_t float2_to_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) __bf16 lev_bf16x2;
  typedef __attribute__((ext_vector_type(2))) float lev_f32x2;
  union { lev_bf16x2 b; uint32_t u; } c;
  c.b = __builtin_convertvector(lev_f32x2{lo, hi}, lev_bf16x2);
  return c.u;
}

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return bf16_to_float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return float_to_bf16(v); }

// ---- wave (64 lanes) and block reductions ---------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// sum over a block of NT threads (NT a multiple of 64, at most 1024); every thread gets the result.
// `red` is shared memory of at least NT/64 floats. Safe to call repeatedly (syncs before reuse).
template <int NT> __device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  if (NT == 64) return v;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) t += red[i];
  return t;
}
template <int NT> __device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  if (NT == 64) return v;
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int i = 1; i < NT / 64; ++i) t = fmaxf(t, red[i]);
  return t;
}

// A workgroup barrier that orders LDS traffic only. __syncthreads() also fences global memory, which makes
// the compiler wait for every outstanding global load before the barrier and so defeats prefetching into
// registers across it. Use this one between "LDS written" and "LDS read" phases when the global loads in
// flight are private to the thread.
__device__ __forceinline__ void lds_barrier() {
  asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// ---- activation functions, in 32-bit --------------------------------------------------------
// x / (1 + 2^t) with the hardware's exp2 and reciprocal (about 1 ulp each): a handful of instructions where expf and
// an IEEE division take thirty. 2^t = inf gives u * 0, the right limit.
__device__ __forceinline__ float lev_sigmoid_mul(float u, float t) {
  return u * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(t));
}

// erf by Abramowitz and Stegun 7.1.26 with the hardware's exp2 and reciprocal: a dozen instructions where erff takes
// several dozen. Absolute error up to 5e-7 in float32 arithmetic: for outputs that are rounded to bfloat16 only.
__device__ __forceinline__ float lev_erf_coarse(float x) {
  const float a = fabsf(x);
  const float t = __builtin_amdgcn_rcpf(1.0f + 0.3275911f * a);
  const float poly = ((((1.061405429f * t - 1.453152027f) * t + 1.421413741f) * t - 0.284496736f) * t + 0.254829592f) * t;
  const float y = 1.0f - poly * __builtin_amdgcn_exp2f(-1.4426950408889634f * a * a);
  return copysignf(y, x);
}
__device__ __forceinline__ float lev_gelu_erf_coarse(float u) { return 0.5f * u * (1.0f + lev_erf_coarse(u * 0.7071067811865476f)); }

__device__ __forceinline__ float lev_activate(float u, int act) {
  constexpr float LOG2E = 1.4426950408889634f;
  switch (act) {
    case LEV_ACT_GELU_TANH: {
      // 0.5 u (1 + tanh z) = u / (1 + exp(-2 z)), z = sqrt(2/pi) (u + 0.044715 u^3): no branches, unlike tanhf
      constexpr float k1 = -2.0f * 0.7978845608028654f * LOG2E, k3 = k1 * 0.044715f;
      return lev_sigmoid_mul(u, u * (k1 + k3 * u * u));
    }
    case LEV_ACT_GELU_ERF: return 0.5f * u * (1.0f + erff(u * 0.7071067811865476f));
    case LEV_ACT_RELU: return fmaxf(u, 0.f);
    case LEV_ACT_SILU: return lev_sigmoid_mul(u, -LOG2E * u);
    case LEV_ACT_QUICK_GELU: return lev_sigmoid_mul(u, -1.702f * LOG2E * u);
    case LEV_ACT_TANH: return tanhf(u);
    default: return u;
  }
}

// ACT >= 0: the activation is known at compile time (no switch per element in a hot loop); ACT < 0: `act` decides
template <int ACT>
__device__ __forceinline__ float lev_activate_as(float u, int act) {
  return lev_activate(u, ACT >= 0 ? ACT : act);
}
