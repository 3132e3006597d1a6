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

// ---------------------------------------------------------------- tokens fed from the device
// token_ids[dst[i]] = source[src[i]]: the tokens that the sampler left on the device for the step before go
// into this step's token ids without a round trip through the host (the host learns them one step late).
// The pairs travel in the launch's arguments, 64 a launch: no memory of their own.
#define FEED_PAIRS 64
struct FeedPairs {
  int dst[FEED_PAIRS];
  int src[FEED_PAIRS];
};

__global__ void feed_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ source, int count, FeedPairs pairs) {
  const int i = threadIdx.x;
  if (i < count) token_ids[pairs.dst[i]] = source[pairs.src[i]];
}

// dst, src: host arrays of `count` indices; every dst below tokens, every src below sources (checked here).
extern "C" int mi_feed_tokens(int* token_ids, int tokens, const int* source, int sources, const int* dst,
                              const int* src, int count, hipStream_t stream) {
  if (count < 0 || tokens <= 0 || sources <= 0 || !token_ids || !source || (count > 0 && (!dst || !src)))
    return ERR_BAD_ARGUMENT;
  for (int i = 0; i < count; ++i)
    if (dst[i] < 0 || dst[i] >= tokens || src[i] < 0 || src[i] >= sources) return ERR_BAD_ARGUMENT;
  for (int first = 0; first < count; first += FEED_PAIRS) {
    FeedPairs pairs = {};
    const int n = count - first < FEED_PAIRS ? count - first : FEED_PAIRS;
    for (int i = 0; i < n; ++i) {
      pairs.dst[i] = dst[first + i];
      pairs.src[i] = src[first + i];
    }
    feed_tokens_kernel<<<1, FEED_PAIRS, 0, stream>>>(token_ids, source, n, pairs);
    RETURN_IF_LAUNCH_FAILED();
  }
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

// The same with four consecutive elements a thread and every load of a row asked for before the
// first is used (d a multiple of 4, at most 256 * 4 * NORM_MAX_ROUNDS).  The order of the sum is
// again fixed by d alone.
#define NORM_MAX_ROUNDS 8
template <typename T> struct Vec4;
template <> struct Vec4<float> { typedef float type __attribute__((ext_vector_type(4))); };
template <> struct Vec4<bf16_t> { typedef __bf16 type __attribute__((ext_vector_type(4))); };

template <typename TD, typename TO, int ROUNDS>
__global__ void __launch_bounds__(256)
add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta0, const TD* __restrict__ delta1,
                       const float* __restrict__ weight, float eps, TO* __restrict__ out,
                       const int* __restrict__ rows, int d) {
  typedef typename Vec4<float>::type f4;
  typedef typename Vec4<TD>::type d4;
  typedef typename Vec4<TO>::type o4;
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  // every load first and none under a condition (a wait counts all loads before it): an absent delta
  // reads the row itself and is dropped, a column past the end reads the last one
  const TD* d0 = delta0 ? delta0 + row * d : reinterpret_cast<const TD*>(hr);
  const TD* d1 = delta1 ? delta1 + row * d : reinterpret_cast<const TD*>(hr);
  f4 v[ROUNDS], w[ROUNDS];
  d4 a[ROUNDS], b[ROUNDS];
  int at[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) at[r] = min(((int)threadIdx.x + r * 256) * 4, d - 4);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) v[r] = *reinterpret_cast<const f4*>(hr + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) a[r] = *reinterpret_cast<const d4*>(d0 + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) b[r] = *reinterpret_cast<const d4*>(d1 + at[r]);
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) w[r] = *reinterpret_cast<const f4*>(weight + at[r]);
  float sum_squares = 0.f;
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const bool mine = ((int)threadIdx.x + r * 256) * 4 < d;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      float value = v[r][j];
      if (delta0) value += (float)a[r][j];
      if (delta1) value += (float)b[r][j];
      v[r][j] = value;
      if (mine) sum_squares += value * value;
    }
    if (mine && !rows && (delta0 || delta1)) *reinterpret_cast<f4*>(hr + at[r]) = v[r];
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
#pragma unroll
    for (int r = 0; r < ROUNDS; ++r) {
      if (((int)threadIdx.x + r * 256) * 4 < d) {
        o4 packed;
#pragma unroll
        for (int j = 0; j < 4; ++j) packed[j] = from_float<TO>(v[r][j] / denominator * w[r][j]);
        *reinterpret_cast<o4*>(o + at[r]) = packed;
      }
    }
  }
}

// ---------------------------------------------------------------- residual add of partial sums + RMSNorm
// The same as add_rmsnorm for a branch that arrives as S float32 slabs [S, T, d] (a product split
// over K): h[row] += sum over the slabs (in slab order), out = h / sqrt(mean(h^2) + eps) * w.
// One workgroup per row; a thread takes four columns at a time and asks for all its slabs at once.
#define PARTIALS_MOST 16
template <typename TO>
__global__ void __launch_bounds__(256)
add_partials_rmsnorm_kernel(float* __restrict__ h, const float* __restrict__ partial, int S, long slab,
                            const float* __restrict__ weight, float eps, TO* __restrict__ out,
                            const int* __restrict__ rows, int d) {
  typedef typename Vec4<float>::type f4;
  typedef typename Vec4<TO>::type o4;
  __shared__ float scratch[16];
  const long out_row = blockIdx.x;
  const long row = rows ? (long)rows[out_row] : out_row;
  float* hr = h + row * d;
  const float* pr = partial + row * d;
  float sum_squares = 0.f;
  for (int column = (int)threadIdx.x * 4; column < d; column += 256 * 4) {
    f4 value = *reinterpret_cast<const f4*>(hr + column);
    f4 parts[PARTIALS_MOST];
#pragma unroll
    for (int s = 0; s < PARTIALS_MOST; ++s) parts[s] = *reinterpret_cast<const f4*>(pr + (long)min(s, S - 1) * slab + column);
#pragma unroll
    for (int s = 0; s < PARTIALS_MOST; ++s)
      if (s < S) {
#pragma unroll
        for (int j = 0; j < 4; ++j) value[j] += parts[s][j];
      }
#pragma unroll
    for (int j = 0; j < 4; ++j) sum_squares += value[j] * value[j];
    *reinterpret_cast<f4*>(hr + column) = value;       // with `rows` the caller passes a copy's row: see the launcher
  }
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)d + eps);
  if (out) {
    TO* o = out + out_row * d;
    for (int column = (int)threadIdx.x * 4; column < d; column += 256 * 4) {
      const f4 value = *reinterpret_cast<const f4*>(hr + column);
      const f4 w = *reinterpret_cast<const f4*>(weight + column);
      o4 packed;
#pragma unroll
      for (int j = 0; j < 4; ++j) packed[j] = from_float<TO>(value[j] / denominator * w[j]);
      *reinterpret_cast<o4*>(o + column) = packed;
    }
  }
}

// With `rows` (a gather: only those rows are normed) the stream itself must stay as it is, and a row may be
// asked for twice; the kernel above writes the sums back, so gathers are refused here and the caller adds
// the partial sums to the stream first (rows == nullptr, out == nullptr) and gathers with mi_add_rmsnorm.
extern "C" int mi_add_partials_rmsnorm(float* h, const float* partial, int S, const float* weight, float eps,
                                       void* out, int out_dtype, const int* rows, int n_rows, int T, int d,
                                       hipStream_t stream) {
  if (!h || !partial || !weight || S < 1 || n_rows <= 0 || T <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  if (rows) return ERR_BAD_ARGUMENT;
  if (S > PARTIALS_MOST || d % 4 != 0) return ERR_UNSUPPORTED_SIZE;
  const long slab = (long)T * d;
  if (out_dtype == DT_BF16)
    add_partials_rmsnorm_kernel<bf16_t><<<n_rows, 256, 0, stream>>>(h, partial, S, slab, weight, eps, (bf16_t*)out, rows, d);
  else if (out_dtype == DT_F32)
    add_partials_rmsnorm_kernel<float><<<n_rows, 256, 0, stream>>>(h, partial, S, slab, weight, eps, (float*)out, rows, d);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

extern "C" int mi_add_rmsnorm(float* h, const void* delta0, const void* delta1, int delta_dtype,
                              const float* weight, float eps, void* out, int out_dtype, const int* rows,
                              int n_rows, int d, hipStream_t stream) {
  if (n_rows <= 0 || d <= 0) return ERR_BAD_ARGUMENT;
  const bool vectors = d % 4 == 0 && d <= 256 * 4 * NORM_MAX_ROUNDS && ((uintptr_t)h % 16) == 0 &&
                       ((uintptr_t)delta0 % 16) == 0 && ((uintptr_t)delta1 % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0 && ((uintptr_t)weight % 16) == 0;
  if (!vectors && (size_t)d * sizeof(float) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  const size_t lds = (size_t)d * sizeof(float);
#define LAUNCH(TD, TO)                                                                                      \
  do {                                                                                                      \
    if (vectors && d <= 1024)                                                                               \
      add_rmsnorm_vec_kernel<TD, TO, 1><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d);        \
    else if (vectors && d <= 2048)                                                                          \
      add_rmsnorm_vec_kernel<TD, TO, 2><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d);        \
    else if (vectors && d <= 4096)                                                                          \
      add_rmsnorm_vec_kernel<TD, TO, 4><<<n_rows, 256, 0, stream>>>(h, (const TD*)delta0, (const TD*)delta1, \
                                                                    weight, eps, (TO*)out, rows, d);        \
    else if (vectors)                                                                                       \
      add_rmsnorm_vec_kernel<TD, TO, NORM_MAX_ROUNDS><<<n_rows, 256, 0, stream>>>(                          \
          h, (const TD*)delta0, (const TD*)delta1, weight, eps, (TO*)out, rows, d);                         \
    else                                                                                                    \
      add_rmsnorm_kernel<TD, TO><<<n_rows, 256, lds, stream>>>(h, (const TD*)delta0, (const TD*)delta1,     \
                                                               weight, eps, (TO*)out, rows, d);             \
  } while (0)
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
// out[t, i] = SiLU(g[t, i]) * u[t, i]      (reference: src/decoder.rs:298-305)
// A row of the input holds [g | u] (tile = 0), or g and u interleaved in tiles:
// [g[0:tile] | u[0:tile] | g[tile:2 tile] | ...], the layout the fused decode kernel wants its
// weight rows in (tile = 8), so that one matrix serves both.
__device__ __forceinline__ long swiglu_gate_at(int i, int I, int tile) {
  return tile == 0 ? i : (long)(i / tile) * 2 * tile + i % tile;
}

template <typename T>
__global__ void swiglu_kernel(const T* __restrict__ gu, long ld, T* __restrict__ out, int I, int tile, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long t = index / I;
  const int i = (int)(index - t * I);
  const long at = swiglu_gate_at(i, I, tile);
  const float gate = to_float(gu[t * ld + at]);
  const float up = to_float(gu[t * ld + at + (tile == 0 ? I : tile)]);
  out[index] = from_float<T>(silu_f(gate) * up);
}

// bfloat16, eight elements a thread (I, ld and the addresses multiples of 8 elements; tile 0 or 8)
typedef __bf16 common_bf16x8 __attribute__((ext_vector_type(8)));
__global__ void __launch_bounds__(256)
swiglu_vec_kernel(const bf16_t* __restrict__ gu, long ld, bf16_t* __restrict__ out, int I, int tile, long total) {
  const long index = ((long)blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (index >= total) return;
  const long t = index / I;
  const int i = (int)(index - t * I);
  const long at = tile == 0 ? i : 2L * i;
  const common_bf16x8 gate = *reinterpret_cast<const common_bf16x8*>(gu + t * ld + at);
  const common_bf16x8 up = *reinterpret_cast<const common_bf16x8*>(gu + t * ld + at + (tile == 0 ? I : 8));
  common_bf16x8 result;
#pragma unroll
  for (int j = 0; j < 8; ++j) result[j] = (bf16_t)(silu_bf16_f((float)gate[j]) * (float)up[j]);
  *reinterpret_cast<common_bf16x8*>(out + index) = result;
}

extern "C" int mi_swiglu(const void* gu, int dtype, long ld, void* out, int T, int I, int tile, hipStream_t stream) {
  if (T <= 0 || I <= 0 || ld < 2L * I || tile < 0 || (tile > 0 && I % tile != 0)) return ERR_BAD_ARGUMENT;
  const long total = (long)T * I;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_BF16 && I % 8 == 0 && ld % 8 == 0 && (tile == 0 || tile == 8) && ((uintptr_t)gu % 16) == 0 &&
      ((uintptr_t)out % 16) == 0) {
    const int vec_blocks = (int)((total / 8 + 255) / 256);
    swiglu_vec_kernel<<<vec_blocks, 256, 0, stream>>>((const bf16_t*)gu, ld, (bf16_t*)out, I, tile, total);
  } else if (dtype == DT_F32)
    swiglu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)gu, ld, (float*)out, I, tile, total);
  else if (dtype == DT_BF16)
    swiglu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)gu, ld, (bf16_t*)out, I, tile, total);
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

// ---------------------------------------------------------------- a cap on the logits
// x <- cap * tanh(x / cap), in place on float32 (reference: src/decoder.rs:4791-4796, after the scaling of the
// logits, :3349-3355)
__global__ void tanh_softcap_kernel(float* __restrict__ x, float cap, float inverse, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) x[index] = cap * tanhf(x[index] * inverse);
}

extern "C" int mi_tanh_softcap(float* x, float cap, long total, hipStream_t stream) {
  if (total <= 0 || !x || !(cap > 0.f)) return ERR_BAD_ARGUMENT;
  const int blocks = (int)((total + 255) / 256);
  tanh_softcap_kernel<<<blocks, 256, 0, stream>>>(x, cap, 1.0f / cap, total);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- bias behind a library product
// out[m, n] = bf16(sums[m, n] + bias[n]): the float32 sums of a bfloat16 product get their float32 bias and are
// rounded once (reference: src/model_weights.rs:530-545 adds the bias to the product's result).
__global__ void add_bias_round_kernel(const float* __restrict__ sums, const float* __restrict__ bias,
                                      bf16_t* __restrict__ out, int N, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index < total) out[index] = (bf16_t)(sums[index] + bias[index % N]);
}

extern "C" int mi_add_bias_round(const float* sums, const float* bias, void* out, int M, int N, hipStream_t stream) {
  if (M <= 0 || N <= 0 || !sums || !bias || !out) return ERR_BAD_ARGUMENT;
  const long total = (long)M * N;
  add_bias_round_kernel<<<(int)((total + 255) / 256), 256, 0, stream>>>(sums, bias, (bf16_t*)out, N, total);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
