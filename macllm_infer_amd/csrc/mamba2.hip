// Mamba2 mixer kernels over a packed batch of lanes (one lane = consecutive tokens of one
// request): causal depthwise conv + SiLU with the saved tail, tail update, the selective
// scan with the per-request state, and the gate (+ grouped RMSNorm).
//
// `u` is the output of the input projection, one row per token, laid out
// [z (E) | x (E) | B (G*N) | C (G*N) | dt (H)]   (reference: src/decoder.rs:2203-2209).
// Per-request state lives in slots: conv tail [slot, K-1, C] in the activation dtype
// (raw, pre-conv rows; reference: src/decoder.rs:2373-2385) and the SSM state
// [slot, H, P, N] in float32 (reference: src/decoder.rs:2269-2294).  A fresh request's slot
// holds zeros.
#include "common.h"

#define CONV_MAX_K 16

// ---------------------------------------------------------------- conv + SiLU
// c[t, ch] = bias[ch] + sum_k w[ch, k] * win[t + k, ch], win = [tail ; this lane's rows];
// w[ch, 0] multiplies the oldest sample (reference: src/decoder.rs:2233-2253, :5948-5950).
template <typename T>
__global__ void conv1d_silu_kernel(const T* __restrict__ u, long ld, int col_offset, int C, int K,
                                   const float* __restrict__ weight, const float* __restrict__ bias,
                                   const T* __restrict__ conv_state, const int* __restrict__ lane_of_token,
                                   const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                                   T* __restrict__ out, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long token = index / C;
  const int channel = (int)(index - token * C);
  const int lane = lane_of_token[token];
  const long lane_start = cu_seqlens[lane];
  const T* tail = conv_state + (long)slot_ids[lane] * (K - 1) * C;
  float sum = bias ? bias[channel] : 0.f;
  for (int k = 0; k < K; ++k) {
    const long source = token - (K - 1) + k;
    float sample;
    if (source >= lane_start)
      sample = to_float(u[source * ld + col_offset + channel]);
    else
      sample = to_float(tail[((K - 1) + (source - lane_start)) * C + channel]);
    sum += weight[channel * K + k] * sample;
  }
  out[index] = from_float<T>(silu_f(sum));
}

// The same for bfloat16 with 8 channels and 4 consecutive token rows per thread: the rows the four
// windows share are loaded once, 16 bytes at a time, together with the taps (contiguous for 8
// channels) and the lanes of the four tokens; no load stands under a condition.  The common case
// (every row of a window belongs to the token's lane) is computed from these; a token among the
// first K-1 of its lane is redone with the rows of the lane's conv tail.
typedef __bf16 conv_bf16x8 __attribute__((ext_vector_type(8)));
typedef float conv_floatx4 __attribute__((ext_vector_type(4)));

template <int K>
__global__ void __launch_bounds__(256)
conv1d_silu_vec_kernel(const bf16_t* __restrict__ u, long ld, int col_offset, int C, int T,
                       const float* __restrict__ weight, const float* __restrict__ bias,
                       const bf16_t* __restrict__ conv_state, const int* __restrict__ lane_of_token,
                       const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                       bf16_t* __restrict__ out) {
  constexpr int ROWS = 4;
  const int vectors = C / 8;
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const long group = index / vectors;
  const int channel = (int)(index - group * vectors) * 8;
  const long t0 = group * ROWS;
  if (t0 >= T) return;
  conv_bf16x8 window[ROWS + K - 1];                 // rows t0-(K-1) .. t0+ROWS-1 of u, clamped into [0, T)
#pragma unroll
  for (int j = 0; j < ROWS + K - 1; ++j) {
    const long row = min(max(t0 - (K - 1) + j, 0L), (long)T - 1);
    window[j] = *reinterpret_cast<const conv_bf16x8*>(u + row * ld + col_offset + channel);
  }
  conv_floatx4 taps[2 * K];                          // weight[channel .. channel+8, 0 .. K): 8K contiguous floats
#pragma unroll
  for (int j = 0; j < 2 * K; ++j) taps[j] = *reinterpret_cast<const conv_floatx4*>(weight + (long)channel * K + 4 * j);
  conv_floatx4 b_lo = {0.f, 0.f, 0.f, 0.f}, b_hi = {0.f, 0.f, 0.f, 0.f};
  if (bias) {
    b_lo = *reinterpret_cast<const conv_floatx4*>(bias + channel);
    b_hi = *reinterpret_cast<const conv_floatx4*>(bias + channel + 4);
  }
  int lane[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) lane[i] = lane_of_token[min(t0 + i, (long)T - 1)];
  int lane_start[ROWS];
#pragma unroll
  for (int i = 0; i < ROWS; ++i) lane_start[i] = cu_seqlens[lane[i]];
  auto tap = [&](int c, int k) { return taps[(c * K + k) / 4][(c * K + k) % 4]; };
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    const long token = t0 + i;
    if (token >= T) break;
    float sum[8];
#pragma unroll
    for (int c = 0; c < 8; ++c) sum[c] = c < 4 ? b_lo[c] : b_hi[c - 4];
    if (token - (K - 1) >= lane_start[i]) {
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int c = 0; c < 8; ++c) sum[c] += tap(c, k) * (float)window[i + k][c];
    } else {
      const bf16_t* tail = conv_state + (long)slot_ids[lane[i]] * (K - 1) * C + channel;
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const long source = token - (K - 1) + k;
        conv_bf16x8 sample = window[i + k];
        if (source < lane_start[i])
          sample = *reinterpret_cast<const conv_bf16x8*>(tail + ((K - 1) + (source - lane_start[i])) * C);
#pragma unroll
        for (int c = 0; c < 8; ++c) sum[c] += tap(c, k) * (float)sample[c];
      }
    }
    conv_bf16x8 result;
#pragma unroll
    for (int c = 0; c < 8; ++c) result[c] = (bf16_t)silu_f(sum[c]);
    *reinterpret_cast<conv_bf16x8*>(out + token * C + channel) = result;
  }
}

extern "C" int mi_conv1d_silu(const void* u, int dtype, long ld, int col_offset, int T, int C, int K,
                              const float* weight, const float* bias, const void* conv_state,
                              const int* lane_of_token, const int* cu_seqlens, const int* slot_ids, void* out,
                              hipStream_t stream) {
  if (T <= 0 || C <= 0 || K <= 0 || K > CONV_MAX_K || ld < col_offset + C) return ERR_BAD_ARGUMENT;
  const long total = (long)T * C;
  const int blocks = (int)((total + 255) / 256);
  const bool aligned = C % 8 == 0 && ld % 8 == 0 && col_offset % 8 == 0 && ((uintptr_t)u % 16) == 0 &&
                       ((uintptr_t)out % 16) == 0 && ((uintptr_t)conv_state % 16) == 0 &&
                       ((uintptr_t)weight % 16) == 0 && ((uintptr_t)bias % 16) == 0;
  if (dtype == DT_BF16 && aligned && K >= 2 && K <= 4) {
    const long threads = (long)((T + 3) / 4) * (C / 8);
    const int vec_blocks = (int)((threads + 255) / 256);
#define CONV_CASE(K_)                                                                                          \
  conv1d_silu_vec_kernel<K_><<<vec_blocks, 256, 0, stream>>>((const bf16_t*)u, ld, col_offset, C, T, weight,   \
                                                             bias, (const bf16_t*)conv_state, lane_of_token,   \
                                                             cu_seqlens, slot_ids, (bf16_t*)out)
    if (K == 2) CONV_CASE(2);
    else if (K == 3) CONV_CASE(3);
    else CONV_CASE(4);
#undef CONV_CASE
    RETURN_IF_LAUNCH_FAILED();
    return 0;
  }
  if (dtype == DT_F32)
    conv1d_silu_kernel<float><<<blocks, 256, 0, stream>>>((const float*)u, ld, col_offset, C, K, weight, bias,
                                                           (const float*)conv_state, lane_of_token, cu_seqlens,
                                                           slot_ids, (float*)out, total);
  else if (dtype == DT_BF16)
    conv1d_silu_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)u, ld, col_offset, C, K, weight, bias,
                                                            (const bf16_t*)conv_state, lane_of_token, cu_seqlens,
                                                            slot_ids, (bf16_t*)out, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- conv tail update
// new tail = last K-1 rows of [old tail ; this lane's rows]; a lane shorter than K-1 keeps
// part of the old tail (reference: src/decoder.rs:2373-2385).  Runs after conv1d_silu.
template <typename T>
__global__ void conv_state_update_kernel(const T* __restrict__ u, long ld, int col_offset, int C, int K,
                                         T* __restrict__ conv_state, const int* __restrict__ cu_seqlens,
                                         const int* __restrict__ slot_ids, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const int lane = (int)(index / C);
  const int channel = (int)(index - (long)lane * C);
  const long lane_start = cu_seqlens[lane];
  const int length = cu_seqlens[lane + 1] - cu_seqlens[lane];
  T* tail = conv_state + (long)slot_ids[lane] * (K - 1) * C;
  T kept[CONV_MAX_K];
  for (int j = 0; j < K - 1; ++j) {
    const int source = length + j;                 // row of the (K-1+length)-row window
    if (source < K - 1)
      kept[j] = tail[(long)source * C + channel];
    else
      kept[j] = u[(lane_start + source - (K - 1)) * ld + col_offset + channel];
  }
  for (int j = 0; j < K - 1; ++j) tail[(long)j * C + channel] = kept[j];
}

extern "C" int mi_conv_state_update(const void* u, int dtype, long ld, int col_offset, int C, int K,
                                    void* conv_state, const int* cu_seqlens, const int* slot_ids,
                                    int num_lanes, hipStream_t stream) {
  if (num_lanes <= 0 || C <= 0 || K <= 0 || K > CONV_MAX_K) return ERR_BAD_ARGUMENT;
  if (K == 1) return 0;
  const long total = (long)num_lanes * C;
  const int blocks = (int)((total + 255) / 256);
  if (dtype == DT_F32)
    conv_state_update_kernel<float><<<blocks, 256, 0, stream>>>((const float*)u, ld, col_offset, C, K,
                                                                 (float*)conv_state, cu_seqlens, slot_ids, total);
  else if (dtype == DT_BF16)
    conv_state_update_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)u, ld, col_offset, C, K,
                                                                  (bf16_t*)conv_state, cu_seqlens, slot_ids, total);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- conv step of single-token lanes
// Row m of u is the one new token of the request in slot_ids[m].  In place on columns
// [col_offset, col_offset + C): u = SiLU(bias + sum_k w[c, k] * window[k]) with window = [tail ; new
// sample]; the tail is rolled by one and takes the sample (the same formula as conv1d_silu and
// conv_state_update for a lane of length one).  One thread per (row, channel); all loads first.
template <typename T, int MAXK>
__global__ void conv_step_kernel(T* __restrict__ u, long ld, int col_offset, int C, int K, const float* __restrict__ weight,
                                 const float* __restrict__ bias, T* __restrict__ conv_state,
                                 const int* __restrict__ slot_ids, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const int m = (int)(index / C);
  const int channel = (int)(index - (long)m * C);
  T* cell = u + (long)m * ld + col_offset + channel;
  T* tail = K > 1 ? conv_state + (long)slot_ids[m] * (K - 1) * C + channel : cell;      // no tail with one tap
  const T sample = *cell;
  T window[MAXK];
  float taps[MAXK];
#pragma unroll
  for (int k = 0; k < MAXK; ++k) {
    window[k] = tail[(long)min(k, max(K - 2, 0)) * C];       // clamped: read, not used, past the tail
    taps[k] = weight[(long)channel * K + min(k, K - 1)];
  }
  float sum = bias ? bias[channel] : 0.f;
#pragma unroll
  for (int k = 0; k < MAXK; ++k) {
    if (k < K - 1) {
      sum += taps[k] * (float)window[k];
      if (k > 0) tail[(long)(k - 1) * C] = window[k];
    } else if (k == K - 1) {
      sum += taps[k] * (float)sample;
    }
  }
  if (K > 1) tail[(long)(K - 2) * C] = sample;
  *cell = (T)silu_f(sum);
}

extern "C" int mi_conv_step(void* u, int dtype, long ld, int col_offset, int M, int C, int K, const float* weight,
                            const float* bias, void* conv_state, const int* slot_ids, hipStream_t stream) {
  if (M <= 0 || C <= 0 || K <= 0 || K > CONV_MAX_K) return ERR_BAD_ARGUMENT;
  const long total = (long)M * C;
  const int blocks = (int)((total + 255) / 256);
#define CONV_STEP(T_, MAXK_)                                                                                  \
  conv_step_kernel<T_, MAXK_><<<blocks, 256, 0, stream>>>((T_*)u, ld, col_offset, C, K, weight, bias, (T_*)conv_state, \
                                                          slot_ids, total)
  if (dtype == DT_F32) {
    if (K <= 4) CONV_STEP(float, 4);
    else CONV_STEP(float, CONV_MAX_K);
  } else if (dtype == DT_BF16) {
    if (K <= 4) CONV_STEP(bf16_t, 4);
    else CONV_STEP(bf16_t, CONV_MAX_K);
  } else {
    return ERR_BAD_ARGUMENT;
  }
#undef CONV_STEP
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- selective scan, token-serial
// Per lane, head h (group g = h / (H/G)), channel p, state row s[N] (float32):
//   delta = softplus(dt + dt_bias[h]);  s = exp(delta*A[h]) * s + delta * x[p] * B[g, :];
//   y[p] = s . C[g, :] + D[h] * x[p]
// (reference: crates/macllm-kernels/src/mamba2.rs:259-288, metal/mamba2_scan.metal:45-77).
// A state row is spread over R lanes of a wavefront (R = power of two <= 64), each holding
// up to SCAN_MAX_PER_THREAD strided elements; 256/R rows per block.
#define SCAN_MAX_PER_THREAD 8

template <typename T>
__global__ void __launch_bounds__(256)
ssm_scan_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt, long dt_ld,
                const float* __restrict__ dt_bias, const float* __restrict__ A, const float* __restrict__ D,
                float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                int H, int P, int N, int G, int R, float* __restrict__ y, long y_ld) {
  const int lane = blockIdx.z;
  const int head = blockIdx.y;
  const int rows_per_block = blockDim.x / R;
  const int row_in_block = threadIdx.x / R;
  const int r = threadIdx.x - row_in_block * R;
  const int p = blockIdx.x * rows_per_block + row_in_block;
  const bool active = p < P;
  const int group = head / (H / G);
  const int E = H * P;
  const long t_begin = cu_seqlens[lane];
  const long t_end = cu_seqlens[lane + 1];
  float* s_row = state + (((long)slot_ids[lane] * H + head) * P + (active ? p : 0)) * N;
  float s[SCAN_MAX_PER_THREAD];
#pragma unroll
  for (int i = 0; i < SCAN_MAX_PER_THREAD; ++i) {
    const int n = r + i * R;
    s[i] = (active && n < N) ? s_row[n] : 0.f;
  }
  const float a = A[head];
  const float bias = dt_bias[head];
  const float skip = D[head];
  for (long t = t_begin; t < t_end; ++t) {
    const T* row = xbc + t * xbc_ld;
    const float delta = softplus_f(to_float(dt[t * dt_ld + head]) + bias);
    const float decay = expf(delta * a);
    const float x = active ? to_float(row[(long)head * P + p]) : 0.f;
    const T* b_row = row + E + (long)group * N;
    const T* c_row = row + E + (long)G * N + (long)group * N;
    const float dx = delta * x;
    float partial = 0.f;
#pragma unroll
    for (int i = 0; i < SCAN_MAX_PER_THREAD; ++i) {
      const int n = r + i * R;
      if (n < N) {
        const float next = decay * s[i] + dx * to_float(b_row[n]);
        s[i] = next;
        partial += next * to_float(c_row[n]);
      }
    }
    for (int offset = R / 2; offset > 0; offset >>= 1) partial += __shfl_xor(partial, offset, WAVE);
    if (active && r == 0) y[t * y_ld + (long)head * P + p] = partial + skip * x;
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < SCAN_MAX_PER_THREAD; ++i) {
      const int n = r + i * R;
      if (n < N) s_row[n] = s[i];
    }
  }
}

extern "C" int mi_ssm_scan(const void* xbc, int dtype, long xbc_ld, const void* dt, long dt_ld,
                           const float* dt_bias, const float* A, const float* D, float* state,
                           const int* cu_seqlens, const int* slot_ids, int num_lanes, int H, int P, int N,
                           int G, float* y, long y_ld, hipStream_t stream) {
  if (num_lanes <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G != 0) return ERR_BAD_ARGUMENT;
  if (N > WAVE * SCAN_MAX_PER_THREAD) return ERR_UNSUPPORTED_SIZE;
  if (H > 65535 || num_lanes > 65535) return ERR_UNSUPPORTED_SIZE;
  int R = 1;
  while (R < N && R < WAVE) R <<= 1;
  const int rows_per_block = 256 / R;
  const dim3 grid((P + rows_per_block - 1) / rows_per_block, H, num_lanes);
  if (dtype == DT_F32)
    ssm_scan_kernel<float><<<grid, 256, 0, stream>>>((const float*)xbc, xbc_ld, (const float*)dt, dt_ld, dt_bias,
                                                      A, D, state, cu_seqlens, slot_ids, H, P, N, G, R, y, y_ld);
  else if (dtype == DT_BF16)
    ssm_scan_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)xbc, xbc_ld, (const bf16_t*)dt, dt_ld,
                                                       dt_bias, A, D, state, cu_seqlens, slot_ids, H, P, N, G, R,
                                                       y, y_ld);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- gate (+ grouped RMSNorm)
// v = y * SiLU(z); with a norm weight, per group of E/G channels:
// out = v / sqrt(mean(v^2) + eps) * w   (gate first, norm after: src/decoder.rs:2350-2367).
// One block per (token, group).
template <typename T>
__global__ void gate_norm_kernel(const float* __restrict__ y, long y_ld, const T* __restrict__ z, long z_ld,
                                 const float* __restrict__ weight, int group_width, float eps,
                                 T* __restrict__ out, long out_ld) {
  __shared__ float scratch[16];
  const long token = blockIdx.x;
  const int group = blockIdx.y;
  const float* y_row = y + token * y_ld + (long)group * group_width;
  const T* z_row = z + token * z_ld + (long)group * group_width;
  T* o_row = out + token * out_ld + (long)group * group_width;
  float sum_squares = 0.f;
  for (int i = threadIdx.x; i < group_width; i += blockDim.x) {
    const float v = y_row[i] * silu_f(to_float(z_row[i]));
    sum_squares += v * v;
    if (!weight) o_row[i] = from_float<T>(v);
  }
  if (!weight) return;
  const float total = block_sum(sum_squares, scratch);
  const float denominator = sqrtf(total / (float)group_width + eps);
  for (int i = threadIdx.x; i < group_width; i += blockDim.x) {
    const float v = y_row[i] * silu_f(to_float(z_row[i]));
    o_row[i] = from_float<T>(v / denominator * weight[(long)group * group_width + i]);
  }
}

extern "C" int mi_gate_norm(const float* y, long y_ld, const void* z, int dtype, long z_ld, const float* weight,
                            int groups, float eps, void* out, long out_ld, int T, int E, hipStream_t stream) {
  if (T <= 0 || E <= 0 || groups <= 0 || E % groups != 0 || groups > 65535) return ERR_BAD_ARGUMENT;
  const int blocks_y = weight ? groups : 1;
  const int width = weight ? E / groups : E;
  const dim3 grid(T, blocks_y);
  if (dtype == DT_F32)
    gate_norm_kernel<float><<<grid, 256, 0, stream>>>(y, y_ld, (const float*)z, z_ld, weight, width, eps,
                                                       (float*)out, out_ld);
  else if (dtype == DT_BF16)
    gate_norm_kernel<bf16_t><<<grid, 256, 0, stream>>>(y, y_ld, (const bf16_t*)z, z_ld, weight, width, eps,
                                                        (bf16_t*)out, out_ld);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
