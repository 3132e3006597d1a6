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

// The same for float32 with four neighbouring channels a thread (16-byte loads of the rows, the taps of the four
// channels in K loads): every channel's sum is formed from the same products in the same order as above.
template <int K>
__global__ void __launch_bounds__(256)
conv1d_silu_f32x4_kernel(const float* __restrict__ u, long ld, int col_offset, int C,
                         const float* __restrict__ weight, const float* __restrict__ bias,
                         const float* __restrict__ conv_state, const int* __restrict__ lane_of_token,
                         const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                         float* __restrict__ out, long total) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const int vectors = C / 4;
  const long token = index / vectors;
  const int channel = (int)(index - token * vectors) * 4;
  const int lane = lane_of_token[token];
  const long lane_start = cu_seqlens[lane];
  const float* tail = conv_state + (long)slot_ids[lane] * (K - 1) * C;
  float4 window[K];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const long source = token - (K - 1) + k;
    // one load, from the rows or from the tail: the address is chosen, not the load
    const float* from = source >= lane_start ? u + source * ld + col_offset + channel
                                             : tail + ((K - 1) + (source - lane_start)) * C + channel;
    window[k] = *reinterpret_cast<const float4*>(from);
  }
  float taps[4 * K];
#pragma unroll
  for (int j = 0; j < K; ++j) {
    const float4 four = *reinterpret_cast<const float4*>(weight + (long)channel * K + 4 * j);
    taps[4 * j] = four.x, taps[4 * j + 1] = four.y, taps[4 * j + 2] = four.z, taps[4 * j + 3] = four.w;
  }
  float4 result;
  float* results = reinterpret_cast<float*>(&result);
#pragma unroll
  for (int c = 0; c < 4; ++c) {
    float sum = bias ? bias[channel + c] : 0.f;
#pragma unroll
    for (int k = 0; k < K; ++k) sum += taps[c * K + k] * reinterpret_cast<const float*>(&window[k])[c];
    results[c] = silu_f(sum);
  }
  *reinterpret_cast<float4*>(out + token * (long)C + channel) = result;
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
  const bool aligned4 = C % 4 == 0 && ld % 4 == 0 && col_offset % 4 == 0 && ((uintptr_t)u % 16) == 0 &&
                        ((uintptr_t)out % 16) == 0 && ((uintptr_t)conv_state % 16) == 0 && ((uintptr_t)weight % 16) == 0;
  if (dtype == DT_F32 && aligned4 && K >= 2 && K <= 4) {
    const long threads = (long)T * (C / 4);
    const int vec_blocks = (int)((threads + 255) / 256);
#define CONV_F32_CASE(K_)                                                                                        \
  conv1d_silu_f32x4_kernel<K_><<<vec_blocks, 256, 0, stream>>>((const float*)u, ld, col_offset, C, weight, bias, \
                                                               (const float*)conv_state, lane_of_token,          \
                                                               cu_seqlens, slot_ids, (float*)out, threads)
    if (K == 2) CONV_F32_CASE(2);
    else if (K == 3) CONV_F32_CASE(3);
    else CONV_F32_CASE(4);
#undef CONV_F32_CASE
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
// A state row is spread over R lanes of a wavefront (R = power of two <= 64), each holding PER neighbouring
// elements (1, 2, 4 or 8: the smallest number that covers N; one load where alignment allows); 256/R rows per block.
//
// The recurrence is serial in the tokens, so what a token costs is what its step waits for.  The tokens of a
// lane come in blocks of up to 16: a block's B, C, x, delta and decay are asked for two blocks ahead by all threads
// of the workgroup, a few elements each and each element once a workgroup, laid in LDS one block ahead, and read
// from there into the registers of the threads that use them, eight tokens (16 / PER) at a time before the first of
// them; softplus and the exponential are taken once a token and head, by a small kernel ahead of the scan.  What
// the R lanes of a row add up for a token's output is added in registers (scan_lanes_sum: a butterfly over the
// lanes in which both partners of every step add the same two numbers), the outputs of a block wait in a register
// of the lane with the token's number and leave with one store a block.  Every token goes through the same
// operations in the same order whatever block it falls into, and in the kernel for steps of single tokens (SINGLE:
// nothing staged, few registers, many workgroups a compute unit): a step of one token and a prompt of thousands
// give a position the same bits.
#define SCAN_MAX_PER_THREAD 8
#define SCAN_BLOCK_ELEMENTS 16      // tokens of a run that goes without a condition, times PER
#define SCAN_BLOCK_TOKENS 16        // tokens of a block that a workgroup stages, at most
#define SCAN_THREAD_PIECES 4        // loads of four elements of B|C that a thread sends for, a block

template <int CONTROL, int ROW_MASK>
__device__ __forceinline__ float scan_dpp(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CONTROL, ROW_MASK, 0xf, false));
}

// The sum of a value over the R lanes of a row (R a power of two, rows at multiples of R), in the last 16 lanes of
// the row (in all of them if R <= 16), the same bits in each of those: within 16 lanes step k adds what the lane's
// group of 2^k lanes holds to what its neighbour group holds, and the lanes of both groups add the same two numbers
// (neighbours within a quad by quad permutation, then the mirrors of half a row and of a row of 16: after the steps
// before, every lane of a group holds the group's sum, so any lane of the neighbour group will do); the sums of the
// 16-lane rows then travel upwards, the last lane of a row to every lane of the next, and of the first two rows to
// the last two: ((s3 + s2) + (s1 + s0)) in a row of 64.  All in the vector pipeline, nothing through LDS.
template <int R>
__device__ __forceinline__ float scan_lanes_sum(float v) {
  if (R >= 2) v += scan_dpp<0xB1, 0xf>(v);            // quad_perm [1, 0, 3, 2]
  if (R >= 4) v += scan_dpp<0x4E, 0xf>(v);            // quad_perm [2, 3, 0, 1]
  if (R >= 8) v += scan_dpp<0x141, 0xf>(v);           // row_half_mirror
  if (R >= 16) v += scan_dpp<0x140, 0xf>(v);          // row_mirror
  if (R >= 32) v += scan_dpp<0x142, 0xa>(v);          // row_bcast15 into rows 1 and 3 (the others add 0)
  if (R >= 64) v += scan_dpp<0x143, 0xc>(v);          // row_bcast31 into rows 2 and 3
  return v;
}

// A barrier of the workgroup for what went through LDS, and nothing else.  __syncthreads() also waits for every load
// from memory that is under way (its fences order all memory), and the loads for the blocks ahead are meant to stay
// under way across the barriers of the block that is being scanned.
__device__ __forceinline__ void scan_lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): this wave's LDS reads and writes are done; vmcnt, expcnt: any
  __builtin_amdgcn_s_barrier();
}

// VECTORS (staged kernel only): B and C come four neighbouring elements a load (N, the row stride and the columns
// of B are multiples of 4 and the rows 16-byte aligned); else element by element.
template <typename T, int PER, int R, bool SINGLE, bool VECTORS>
__global__ void __launch_bounds__(256, 2)          // two workgroups a compute unit at least
ssm_scan_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt, long dt_ld,
                const float* __restrict__ dt_bias, const float* __restrict__ A, const float* __restrict__ D,
                float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                int H, int P, int N, int G, int block_tokens, const float* __restrict__ delta_decay,
                float* __restrict__ y, long y_ld) {
  constexpr int TB = PER == 1 ? SCAN_BLOCK_ELEMENTS / 2 : SCAN_BLOCK_ELEMENTS / PER;    // tokens of a run that goes without a condition
  constexpr int ROWS = 256 / R;                        // rows of a workgroup
  constexpr int SUM_LANES = R < 16 ? R : 16;           // the last lanes of a row, which hold its sums
  constexpr int FIRST_SUM_LANE = R - SUM_LANES;
  extern __shared__ __align__(16) float staged_l[];    // the staged kernel's two blocks of operands
  const int lane = blockIdx.z;
  const int head = blockIdx.y;
  const int tid = threadIdx.x;
  const int row_in_block = tid / R;
  const int r = tid % R;
  const int p0 = blockIdx.x * ROWS;
  const int p = p0 + row_in_block;
  const bool active = p < P;
  const int group = head / (H / G);
  const int E = H * P;
  const long t_begin = cu_seqlens[lane];
  const long t_end = cu_seqlens[lane + 1];
  if (t_end <= t_begin) return;                        // a lane without tokens (padding of a fixed capacity)
  float* s_row = state + (((long)slot_ids[lane] * H + head) * P + (active ? p : 0)) * N;
  float s[PER];
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int n = r * PER + i;
    s[i] = (active && n < N) ? s_row[n] : 0.f;
  }
  const float skip = D[head];
  // the state is waited for here, once: left to the compiler, the wait lands inside the loop over the blocks, where
  // it also waits for the loads of the blocks ahead, every time round
  __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0)
  const long b_col = E + (long)group * N;
  const long c_col = E + (long)G * N + (long)group * N;
  const long x_col = (long)head * P + (active ? p : 0);
  float* y_mine = y + (long)head * P + (active ? p : 0);

  if (SINGLE) {
    const float a = A[head];
    const float bias = dt_bias[head];
    for (long t = t_begin; t < t_end; ++t) {
      const T* row = xbc + t * xbc_ld;
      const float delta = softplus_f(to_float(dt[t * dt_ld + head]) + bias);
      const float decay = expf(delta * a);
      const float x = active ? to_float(row[x_col]) : 0.f;
      const float dx = delta * x;
      float partial = 0.f;
#pragma unroll
      for (int i = 0; i < PER; ++i) {
        const int n = r * PER + i;
        if (n < N) {
          const float next = fmaf(decay, s[i], dx * to_float(row[b_col + n]));
          s[i] = next;
          partial = fmaf(next, to_float(row[c_col + n]), partial);
        }
      }
      const float sum = scan_lanes_sum<R>(partial);
      if (r == R - 1 && active) y_mine[t * y_ld] = fmaf(skip, x, sum);
    }
  } else {
    // A block's operands are brought in by all 256 threads: a thread lays its share of block b + 1 in LDS at the
    // start of the round of block b, asks for its share of block b + 2 into the same registers, stores the outputs
    // of block b - 1, and then works on block b.  Its loads so have a block's time to arrive, and the wait for
    // them (which a wave can only state for all it has asked of memory at once, stores included) never meets a
    // load or a store of a moment ago.  Every element comes in once a workgroup: the rows of a head, and the
    // heads of a group, read the same B and C.
    const int row_floats = 2 * N;
    float* b_l = staged_l;                                      // [2][block_tokens][2 N]: B then C of a token
    float* x_l = b_l + 2 * block_tokens * row_floats;           // [2][block_tokens][ROWS]
    float* dd_l = x_l + 2 * block_tokens * ROWS;                // [2][block_tokens][2]: delta, decay
    typedef T pieces __attribute__((ext_vector_type(4)));
    const int pieces_a_row = (row_floats + 3) / 4;
    const bool whole_rows = N == R * PER;                       // no lane of a row is idle
    float staged_bc[SCAN_THREAD_PIECES][4], staged_x = 0.f, staged_dd = 0.f;
    // where this thread's pieces lie in a block (the same for every block: worked out once, a division each)
    int piece_token[SCAN_THREAD_PIECES], piece_col[SCAN_THREAD_PIECES];
#pragma unroll
    for (int j = 0; j < SCAN_THREAD_PIECES; ++j) {
      const int index = tid + j * 256;
      piece_token[j] = index / pieces_a_row;
      piece_col[j] = (index - piece_token[j] * pieces_a_row) * 4;
    }
    const int x_token = tid / ROWS, x_row = tid % ROWS;
    // this thread's share of block `block` of the lane into its registers (nothing if the lane has no such block)
    auto fetch = [&](int block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)max(0L, min((long)block_tokens, t_end - t0));
      if (count <= 0) return;
#pragma unroll
      for (int j = 0; j < SCAN_THREAD_PIECES; ++j) {
        const int token = min(piece_token[j], count - 1);           // a piece past the block reads its last token, unused
        const int col = piece_col[j];
        if (VECTORS) {
          // B and C of a group lie apart in a row: columns N .. 2 N of the staged row are C
          const pieces four = *reinterpret_cast<const pieces*>(xbc + (t0 + token) * xbc_ld + (col < N ? b_col + col : c_col + (col - N)));
#pragma unroll
          for (int i = 0; i < 4; ++i) staged_bc[j][i] = to_float<T>(four[i]);
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) {                         // element by element: a piece may straddle B and C
            const int at = min(col + i, row_floats - 1);
            staged_bc[j][i] = to_float(xbc[(t0 + token) * xbc_ld + (at < N ? b_col + at : c_col + (at - N))]);
          }
        }
      }
      const int row = p0 + x_row;
      staged_x = row < P ? to_float(xbc[(t0 + min(x_token, count - 1)) * xbc_ld + (long)head * P + row]) : 0.f;
      staged_dd = delta_decay[((t0 + min(tid >> 1, count - 1)) * H + head) * 2 + (tid & 1)];
    };
    // this thread's registers (block `block`) into LDS
    auto lay_down = [&](int block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)max(0L, min((long)block_tokens, t_end - t0));
      if (count <= 0) return;
      const int phase = block & 1;
      float* rows_l = b_l + phase * block_tokens * row_floats;
#pragma unroll
      for (int j = 0; j < SCAN_THREAD_PIECES; ++j) {
        const int token = piece_token[j];
        const int col = piece_col[j];
        if (token < count) {
          float* to = rows_l + token * row_floats + col;
          if (VECTORS) {
            *reinterpret_cast<float4*>(to) = make_float4(staged_bc[j][0], staged_bc[j][1], staged_bc[j][2], staged_bc[j][3]);
          } else {
#pragma unroll
            for (int i = 0; i < 4; ++i)
              if (col + i < row_floats) to[i] = staged_bc[j][i];
          }
        }
      }
      if (x_token < count) x_l[phase * block_tokens * ROWS + tid] = staged_x;
      if (tid < 2 * count) dd_l[phase * block_tokens * 2 + tid] = staged_dd;
    };
    // the outputs of the block before: token i of the block waits in the i-th of the row's lanes that hold sums
    // (block_tokens <= SUM_LANES)
    float kept = 0.f;
    long kept_t0 = 0;
    int kept_count = 0;
    auto store_kept = [&]() {
      if (r >= FIRST_SUM_LANE && r - FIRST_SUM_LANE < kept_count && active) y_mine[(kept_t0 + r - FIRST_SUM_LANE) * y_ld] = kept;
    };
    fetch(0);
    lay_down(0);
    fetch(1);
    const int blocks = (int)((t_end - t_begin + block_tokens - 1) / block_tokens);
    for (int block = 0; block < blocks; ++block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)min((long)block_tokens, t_end - t0);
      const int phase = block & 1;
      scan_lds_barrier();                   // this block's operands are laid down, and everybody has read the block
                                            // before the last: its place may be written
      if (block > 0) {
        lay_down(block + 1);
        fetch(block + 2);
        store_kept();
      }
      const float* rows_l = b_l + phase * block_tokens * row_floats;
      const float* x_now = x_l + phase * block_tokens * ROWS + row_in_block;
      const float* dd_now = dd_l + phase * block_tokens * 2;
      const float* mine_l = rows_l + min(r * PER, N - PER > 0 ? N - PER : 0);    // this thread's columns of B (C: N further)
      // runs of TB tokens of a row whose lanes all hold PER elements go without a condition: straight code that
      // asks LDS for the run's operands at once; what is left of a block, and rows with idle lanes, take the
      // guarded loop
      int done = 0;
      if (whole_rows) {
        for (; done + TB <= count; done += TB) {
          float b[TB][PER], c[TB][PER], decay[TB], dx[TB];
#pragma unroll
          for (int token = 0; token < TB; ++token) {
            const float2 delta_and_decay = *reinterpret_cast<const float2*>(dd_now + (done + token) * 2);
            decay[token] = delta_and_decay.y;
            dx[token] = delta_and_decay.x * x_now[(done + token) * ROWS];
#pragma unroll
            for (int i = 0; i < PER; ++i) {
              b[token][i] = mine_l[(done + token) * row_floats + i];
              c[token][i] = mine_l[(done + token) * row_floats + N + i];
            }
          }
          // the x of the token whose output this lane keeps (any token of the run for the other lanes)
          const int my_token = done + ((r - FIRST_SUM_LANE - done) & (TB - 1));
          const float my_x = x_now[my_token * ROWS];
          float my_sum = 0.f;
#pragma unroll
          for (int token = 0; token < TB; ++token) {
            float partial = 0.f;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
              const float next_s = fmaf(decay[token], s[i], dx[token] * b[token][i]);
              s[i] = next_s;
              partial = fmaf(next_s, c[token][i], partial);
            }
            const float sum = scan_lanes_sum<R>(partial);
            my_sum = my_token == done + token ? sum : my_sum;
          }
          kept = (r >= FIRST_SUM_LANE + done && r < FIRST_SUM_LANE + done + TB) ? fmaf(skip, my_x, my_sum) : kept;
        }
      }
      for (int token = done; token < count; ++token) {
        const float decay = dd_now[token * 2 + 1];
        const float x = x_now[token * ROWS];
        const float dx = dd_now[token * 2] * x;
        float partial = 0.f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
          const int n = r * PER + i;
          if (n < N) {
            const float next_s = fmaf(decay, s[i], dx * rows_l[token * row_floats + n]);
            s[i] = next_s;
            partial = fmaf(next_s, rows_l[token * row_floats + N + n], partial);
          }
        }
        const float out = fmaf(skip, x, scan_lanes_sum<R>(partial));
        kept = r == FIRST_SUM_LANE + token ? out : kept;
      }
      kept_t0 = t0;
      kept_count = count;
      if (block == 0) {                     // the first round lays the second block down behind its own work
        lay_down(1);
        fetch(2);
      }
    }
    store_kept();
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int n = r * PER + i;
      if (n < N) s_row[n] = s[i];
    }
  }
}

// delta = softplus(dt + dt_bias[h]) and decay = exp(delta * A[h]) of every token and head, once, for the staged scan
// (the kernel for steps of single tokens forms the same two values from the same operations itself).
template <typename T>
__global__ void scan_delta_decay_kernel(const T* __restrict__ dt, long dt_ld, const float* __restrict__ dt_bias,
                                        const float* __restrict__ A, int H, long total, float* __restrict__ out) {
  const long index = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (index >= total) return;
  const long token = index / H;
  const int head = (int)(index - token * H);
  const float delta = softplus_f(to_float(dt[token * dt_ld + head]) + dt_bias[head]);
  out[2 * index] = delta;
  out[2 * index + 1] = expf(delta * A[head]);
}

template <typename T, int PER, int R>
static void launch_scan(dim3 grid, size_t bytes, hipStream_t stream, bool single, bool vectors, const void* xbc,
                        long xbc_ld, const void* dt, long dt_ld, const float* dt_bias, const float* A, const float* D,
                        float* state, const int* cu_seqlens, const int* slot_ids, int H, int P, int N, int G,
                        int block_tokens, const float* delta_decay, float* y, long y_ld) {
#define SCAN_ARGUMENTS                                                                                              \
  (const T*)xbc, xbc_ld, (const T*)dt, dt_ld, dt_bias, A, D, state, cu_seqlens, slot_ids, H, P, N, G, block_tokens, \
      delta_decay, y, y_ld
  if (single) ssm_scan_kernel<T, PER, R, true, false><<<grid, 256, bytes, stream>>>(SCAN_ARGUMENTS);
  else if (vectors) ssm_scan_kernel<T, PER, R, false, true><<<grid, 256, bytes, stream>>>(SCAN_ARGUMENTS);
  else ssm_scan_kernel<T, PER, R, false, false><<<grid, 256, bytes, stream>>>(SCAN_ARGUMENTS);
#undef SCAN_ARGUMENTS
}

// longest: an upper bound of the tokens of a lane (0: unknown); a step whose lanes all hold one token takes the
// kernel without staging.  delta_decay: float32 [T, H, 2], a work area that the staged kernel needs (T: the tokens
// of all lanes); it may be null when longest == 1.
extern "C" int mi_ssm_scan(const void* xbc, int dtype, long xbc_ld, const void* dt, long dt_ld,
                           const float* dt_bias, const float* A, const float* D, float* state,
                           const int* cu_seqlens, const int* slot_ids, int num_lanes, int longest, int H, int P, int N,
                           int G, float* delta_decay, long tokens, float* y, long y_ld, hipStream_t stream) {
  if (num_lanes <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G != 0) return ERR_BAD_ARGUMENT;
  if (N > WAVE * SCAN_MAX_PER_THREAD) return ERR_UNSUPPORTED_SIZE;
  if (H > 65535 || num_lanes > 65535) return ERR_UNSUPPORTED_SIZE;
  if (dtype != DT_F32 && dtype != DT_BF16) return ERR_BAD_ARGUMENT;
  int R = 1;
  while (R < N && R < WAVE) R <<= 1;
  const int rows_per_block = 256 / R;
  const dim3 grid((P + rows_per_block - 1) / rows_per_block, H, num_lanes);
  const int per_needed = (N + R - 1) / R;
  const int per = per_needed <= 1 ? 1 : per_needed <= 2 ? 2 : per_needed <= 4 ? 4 : 8;
  const bool single = longest == 1;
  if (!single && (!delta_decay || tokens <= 0)) return ERR_BAD_ARGUMENT;
  // tokens of a block: no more than R (a block's x values, one a row and token, are one a thread, and its outputs
  // wait one a lane of the row), and B and C of a block no more than SCAN_THREAD_PIECES loads of four elements a thread
  int block_tokens = SCAN_BLOCK_TOKENS;
  if (block_tokens > R) block_tokens = R;
  while (block_tokens > 1 && (long)block_tokens * ((2 * N + 3) / 4) > 256L * SCAN_THREAD_PIECES) block_tokens /= 2;
  const size_t bytes = single ? 0 : 2 * (size_t)block_tokens * (2 * N + rows_per_block + 2) * sizeof(float);
  // four elements a load: every head's and group's columns of B and C start at multiples of 4
  const bool vectors = !single && N % 4 == 0 && xbc_ld % 4 == 0 && ((long)H * P) % 4 == 0 &&
                       ((uintptr_t)xbc % (dtype == DT_F32 ? 16 : 8)) == 0;
  if (!single) {
    const long total = tokens * H;
    const int blocks = (int)((total + 255) / 256);
    if (dtype == DT_F32)
      scan_delta_decay_kernel<float><<<blocks, 256, 0, stream>>>((const float*)dt, dt_ld, dt_bias, A, H, total, delta_decay);
    else
      scan_delta_decay_kernel<bf16_t><<<blocks, 256, 0, stream>>>((const bf16_t*)dt, dt_ld, dt_bias, A, H, total, delta_decay);
    RETURN_IF_LAUNCH_FAILED();
  }
#define SCAN_CASE(PER_, R_)                                                                                          \
  if (per == PER_ && R == R_) {                                                                                      \
    if (dtype == DT_F32)                                                                                             \
      launch_scan<float, PER_, R_>(grid, bytes, stream, single, vectors, xbc, xbc_ld, dt, dt_ld, dt_bias, A, D,      \
                                   state, cu_seqlens, slot_ids, H, P, N, G, block_tokens, delta_decay, y, y_ld);    \
    else                                                                                                             \
      launch_scan<bf16_t, PER_, R_>(grid, bytes, stream, single, vectors, xbc, xbc_ld, dt, dt_ld, dt_bias, A, D,     \
                                    state, cu_seqlens, slot_ids, H, P, N, G, block_tokens, delta_decay, y, y_ld);   \
  }
  // a row narrower than a wave has one element a lane; a row of 64 lanes 1, 2, 4 or 8
  SCAN_CASE(1, 1) SCAN_CASE(1, 2) SCAN_CASE(1, 4) SCAN_CASE(1, 8) SCAN_CASE(1, 16) SCAN_CASE(1, 32) SCAN_CASE(1, 64)
  SCAN_CASE(2, 64) SCAN_CASE(4, 64) SCAN_CASE(8, 64)
#undef SCAN_CASE
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
