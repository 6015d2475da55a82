// Shared helpers of the sequence-mixer / MoE kernels (extension `_C_mixers`).
//
// Every kernel is instantiated for fp32 and bf16 activations (`T` = float or
// ft::bf16_raw); statistics, scores, recurrent state and gates are fp32 in both.
// Launchers take `int bf16` flags and void pointers, and the caller's stream.
#pragma once

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "ft_common.h"

namespace mx {

using bf16_t = ft::bf16_raw;

__device__ __forceinline__ float ld(const float* p, long i) { return p[i]; }
__device__ __forceinline__ float ld(const bf16_t* p, long i) { return ft::bf16_to_f32(p[i]); }
__device__ __forceinline__ void st(float* p, long i, float v) { p[i] = v; }
__device__ __forceinline__ void st(bf16_t* p, long i, float v) { p[i] = ft::f32_to_bf16(v); }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }

// softplus with the usual linear branch for large arguments
__device__ __forceinline__ float softplusf_(float x) { return x > 20.0f ? x : log1pf(expf(x)); }

// sum over a block of NT threads (NT multiple of 64, <= 1024); every thread gets it
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = ft::wave_sum(v);
  constexpr int NW = NT / 64;
  if constexpr (NW == 1) return v;
  __syncthreads();   // red may still be read from a previous call
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float s = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) s += red[w];
  return s;
}

}  // namespace mx

#define MX_DISPATCH_T(bf16, ...)            \
  do {                                      \
    if (bf16) {                             \
      using T = ::mx::bf16_t;               \
      __VA_ARGS__;                          \
    } else {                                \
      using T = float;                      \
      __VA_ARGS__;                          \
    }                                       \
  } while (0)
