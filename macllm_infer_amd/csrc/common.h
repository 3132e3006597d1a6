// Shared device helpers for the gfx950 kernels: element types, wave and block
// reductions, launch checking.  Wavefronts are 64 lanes wide.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define WAVE 64

typedef __bf16 bf16_t;

// dtype codes used by every entry point
#define DT_F32 0
#define DT_BF16 1

template <typename T> __device__ __forceinline__ float to_float(T v);
template <> __device__ __forceinline__ float to_float<float>(float v) { return v; }
template <> __device__ __forceinline__ float to_float<bf16_t>(bf16_t v) { return (float)v; }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float v) { return (bf16_t)v; }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) v += __shfl_xor(v, offset, WAVE);
  return v;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) v = fmaxf(v, __shfl_xor(v, offset, WAVE));
  return v;
}

// Sum over a block of up to 1024 threads; every thread gets the result.
// `scratch` must hold at least 16 floats of LDS and may be reused after the call.
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int waves = (blockDim.x + WAVE - 1) / WAVE;
  v = wave_sum(v);
  __syncthreads();
  if (lane == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
  for (int i = 0; i < waves; ++i) total += scratch[i];
  return total;
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + expf(-x)); }
// the same with the hardware's exponential and reciprocal (a few float32 ulps): for results that are rounded to
// bfloat16 at once
__device__ __forceinline__ float silu_bf16_f(float x) { return x * __frcp_rn(1.0f + __expf(-x)); }

// max(x,0) + log1p(exp(-|x|)): finite for any finite x.
__device__ __forceinline__ float softplus_f(float x) { return fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))); }

#define RETURN_IF_LAUNCH_FAILED()                 \
  do {                                            \
    hipError_t launch_error_ = hipGetLastError(); \
    if (launch_error_ != hipSuccess) return (int)launch_error_; \
  } while (0)

// Argument errors reported by entry points before anything is launched.
#define ERR_BAD_ARGUMENT (-1)
#define ERR_UNSUPPORTED_SIZE (-2)
