// Embedding gather, residual add + RMSNorm, SwiGLU, logit scaling.
// The residual stream is float32; activations are float32 or bfloat16.
#include "common.h"

// ---------------------------------------------------------------- embedding
// h[t, :] = table[ids[t], :] * multiplier        (reference: src/decoder.rs:3194-3197)
template <typename T>
__global__ void embed_kernel(const int* __restrict__ ids, const T* __restrict__ table, float multiplier,
                             float* __restrict__ h, int d) {
  const long token = blockIdx.x;
  const T* row = table + (long)ids[token] * d;
  float* out = h + token * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) out[i] = to_float(row[i]) * multiplier;
}

extern "C" int mi_embed(const int* ids, const void* table, int table_dtype, float multiplier, float* h,
                        int T, int d, hipStream_t stream) {
  if (T <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if (table_dtype == DT_F32)
    embed_kernel<float><<<T, 256, 0, stream>>>(ids, (const float*)table, multiplier, h, d);
  else if (table_dtype == DT_BF16)
    embed_kernel<bf16_t><<<T, 256, 0, stream>>>(ids, (const bf16_t*)table, multiplier, h, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- add + rmsnorm
// For each processed row r:  v = h[r] (+ delta0[r]) (+ delta1[r]);  if update: h[r] = v;
// out[i] = v / sqrt(mean(v^2) + eps) * weight.
// With `rows` the kernel processes h[rows[i]] and writes out[i] (h is not updated).
// The sum of squares is accumulated in float32 in an order fixed by (d, blockDim) alone,
// so a row's result does not depend on what else is in the batch.
template <typename TD, typename TO>
__global__ void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta0,
                                   const TD* __restrict__ delta1, const float* __restrict__ weight, float eps,
                                   TO* __restrict__ out, const int* __restrict__ rows, int d) {
  extern __shared__ float row_values[];
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  float sum_squares = 0.f;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float v = hr[i];
    if (delta0) v += to_float(delta0[row * d + i]);
    if (delta1) v += to_float(delta1[row * d + i]);
    if (!rows && (delta0 || delta1)) hr[i] = v;
    row_values[i] = v;
    sum_squares += v * v;
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
    for (int i = threadIdx.x; i < d; i += blockDim.x)
      o[i] = from_float<TO>(row_values[i] / denominator * weight[i]);
  }
}

extern "C" int mi_add_rmsnorm(float* h, const void* delta0, const void* delta1, int delta_dtype,
                              const float* weight, float eps, void* out, int out_dtype, const int* rows,
                              int n_rows, int d, hipStream_t stream) {
  if (n_rows <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if ((size_t)d * sizeof(float) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  const size_t lds = (size_t)d * sizeof(float);
#define LAUNCH(TD, TO)                                                                               \
  add_rmsnorm_kernel<TD, TO><<<n_rows, 256, lds, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                            weight, eps, (TO*)out, rows, d)
  if (delta_dtype == DT_F32 && out_dtype == DT_F32) LAUNCH(float, float);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_BF16) LAUNCH(bf16_t, bf16_t);
  else if (delta_dtype == DT_F32 && out_dtype == DT_BF16) LAUNCH(float, bf16_t);
  else if (delta_dtype == DT_BF16 && out_dtype == DT_F32) LAUNCH(bf16_t, float);
  else return ERR_BAD_ARGUMENT;
#undef LAUNCH
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- SwiGLU
// out[t, i] = SiLU(gu[t, i]) * gu[t, I + i]      (reference: src/decoder.rs:298-305)
template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, long ld, T* __restrict__ out, int I, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long t = index / I;
  const int i = (int)(index - t * I);
  const float gate = to_float(gu[t * ld + i]);
  const float up = to_float(gu[t * ld + I + i]);
  out[index] = from_float<T>(silu_f(gate) * up);
}

extern "C" int mi_swiglu(const void* gu, int dtype, long ld, void* out, int T, int I, hipStream_t stream) {
  if (T <= 0 || I <= 0 || ld < 2L * I) return ERR_BAD_ARGUMENT;
  const long total = (long)T * I;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, ld, (float*)out, I, total);
  else if (dtype == DT_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, ld, (bf16_t*)out, I, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- logits to float32
// out[i] = (float)in[i] * multiplier              (reference: src/decoder.rs:3349-3357)
template <typename T>
__global__ void scale_to_f32_kernel(const T* __restrict__ in, float multiplier, float* __restrict__ out, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) out[index] = to_float(in[index]) * multiplier;
}

extern "C" int mi_scale_to_f32(const void* in, int dtype, float multiplier, float* out, long total,
                               hipStream_t stream) {
  if (total <= 0) return ERR_BAD_ARGUMENT;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_F32)
    scale_to_f32_kernel<float><<<blocks, 256, 0, stream>>>((const float*)in, multiplier, out, total);
  else if (dtype == DT_BF16)
    scale_to_f32_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)in, multiplier, out, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
