// Shared device helpers for the gfx950 kernels: wave64 reductions, bfloat16 access,
// launch-error reporting.  Every entry point is `extern "C"`, takes raw device pointers
// and a stream, and returns the hipError_t of its launches (0 = success).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define MF_WAVE 64
#define MF_PAGE 64   // tokens per cache page; pages are [n_kv_heads][MF_PAGE][head_dim]

typedef __bf16 bf16;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

#define MF_API extern "C" __attribute__((visibility("default")))

static inline int mf_launch_status() { return (int)hipGetLastError(); }

__device__ __forceinline__ float to_f32(float v) { return v; }
__device__ __forceinline__ float to_f32(bf16 v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_f32(float v);
template <> __device__ __forceinline__ float from_f32<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_f32<bf16>(float v) { return (bf16)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MF_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MF_WAVE));
  return v;
}

// Sum over a block of NT threads (NT a multiple of 64, at most 1024); every thread gets
// the result.  `scratch` holds NT/64 floats.  The order of additions is fixed, so two
// runs give the same bits.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < NT / 64; ++i) t += scratch[i];
  return t;
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float* scratch) {
  v = wave_max(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) scratch[w] = v;
  __syncthreads();
  float t = scratch[0];
#pragma unroll
  for (int i = 1; i < NT / 64; ++i) t = fmaxf(t, scratch[i]);
  return t;
}
