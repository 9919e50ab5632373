// Sampling without any allocation: a second entry point beside lev_sample.
//
// This entry point has no counterpart in the reference. It is for callers that cannot allocate device memory:
// code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc. lev_sample takes the
// memory for its per-part candidates (lev_sample_workspace(rows) bytes) from the caller; lev_sample_static keeps
// it in a file-scope __device__ array of the library instead and calls neither hipMalloc / hipFree nor any
// allocating library routine. The caller still passes inputs and outputs; arguments and results are those of
// lev_sample (same kernels, bit-identical tokens and log-probabilities).
//
// Limits and rules:
//   * at most LEV_SAMPLE_STATIC_MAX_ROWS rows per call (the array holds rows x 64 parts x 4 floats = 256 KiB
//     on every GPU the library runs on, until the process ends); more rows are refused with an error;
//   * every call on a GPU uses that GPU's one array, so calls that overlap on one GPU (two streams, two
//     threads) race: keep them on one stream or order them with events. The array keeps the last call's contents;
//     nothing in it has to start at zero, the first kernel overwrites every slot the second one reads;
//   * lev_sample_static_init() looks up the array's device address for the current device (hipGetSymbolAddress,
//     once per device). Call it once per device at set-up, outside any graph capture; a call of lev_sample_static on
//     a device that was not initialised does it first.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LEV_SAMPLE_STATIC_MAX_ROWS 256

extern "C" int lev_sample_static_init();
extern "C" int lev_sample_static_max_rows();
extern "C" int lev_sample_static(const float* logits, long row_stride, const float* temperature, const uint32_t* keys,
                                 const int* positions, int* tokens, float* logprobs, int R, int V, hipStream_t stream);
