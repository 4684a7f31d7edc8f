// Shared device helpers for the gfx950 kernels: storage types, conversions,
// wavefront reductions and the error convention of the C entry points.
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

#define PAE_WAVE 64

// dtype codes shared with the Python side
#define PAE_F32 0
#define PAE_BF16 1

typedef __hip_bfloat16 bf16_t;

// Every entry point returns 0 on success.  On refusal it returns a negative code
// and leaves a message that pae_last_error() hands to the caller.
extern "C" const char* pae_last_error();
int pae_fail(const char* fmt, ...);
int pae_check_launch(const char* what);

#define PAE_REQUIRE(cond, ...)                 \
  do {                                         \
    if (!(cond)) return pae_fail(__VA_ARGS__); \
  } while (0)

__device__ __forceinline__ float to_f32(float x) { return x; }
__device__ __forceinline__ float to_f32(bf16_t x) { return __bfloat162float(x); }

template <typename T>
__device__ __forceinline__ T from_f32(float x);
template <>
__device__ __forceinline__ float from_f32<float>(float x) { return x; }
template <>
__device__ __forceinline__ bf16_t from_f32<bf16_t>(float x) { return __float2bfloat16(x); }

// Value of x after a round trip through storage type T (round-to-nearest-even).
template <typename T>
__device__ __forceinline__ float round_to(float x) { return to_f32(from_f32<T>(x)); }

// A vector parameter (norm weight, bias) may be stored in float32 even when
// activations are bfloat16: `is_f32` says which.
__device__ __forceinline__ float load_param(const void* p, int is_f32, int64_t i) {
  return is_f32 ? ((const float*)p)[i] : __bfloat162float(((const bf16_t*)p)[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = PAE_WAVE / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, PAE_WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = PAE_WAVE / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, PAE_WAVE));
  return v;
}

// Sum over a block of `NW` wavefronts in a fixed order: lanes by butterfly,
// then wave partials 0..NW-1 in sequence.  `scratch` holds NW floats in LDS.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / PAE_WAVE;
  if ((threadIdx.x & (PAE_WAVE - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) total += scratch[w];
  __syncthreads();
  return total;
}
