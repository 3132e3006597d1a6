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
// A state row is spread over R lanes of a wavefront (R = power of two <= 64), each holding PER neighbouring
// elements (1, 2, 4 or 8: the smallest number that covers N; one load where alignment allows); 256/R rows per block.
//
// The recurrence is serial in the tokens, so what a token costs is what its step waits for.  The tokens of a
// lane come in blocks of 16 / PER (8 at most): a block's B, C, x and dt are asked for four blocks ahead, each element
// once a workgroup, laid in LDS one block ahead, and read from there into the registers of the threads that use them
// before the block's first token; softplus and the exponential are taken once a token, not once a thread; what the lanes of a row add up for a
// token's output goes to LDS and is added up for the whole block at its end, in the order of the lanes (a pass
// over the wave for every token costs more than the token's own arithmetic).  Every token goes through the same
// operations in the same order whatever block it falls into, and in the kernel for steps of single tokens
// (SINGLE: nothing staged, few registers, many workgroups a compute unit): a step of one token and a prompt of
// thousands give a position the same bits.
#define SCAN_MAX_PER_THREAD 8
#define SCAN_BLOCK_ELEMENTS 16      // tokens of a block times PER
#define SCAN_STAGE_PIECES (SCAN_BLOCK_ELEMENTS / 2)   // loads of four elements of B|C a lane of the wave whose turn it is sends for

// The shares of a row's R lanes as one sum: four quarters of the row (two halves of two lanes, one lane), each
// added up in the order of its lanes, then ((q0 + q1) + q2) + q3.  scan_part_sum is one quarter; scan_row_sum all
// of it in one thread; four threads that take a quarter each and then add the four in that order get the same bits.
__device__ __forceinline__ float scan_part_sum(const float* shares, int R, int part) {
  const int width = R >= 4 ? R / 4 : 1;
  const float* mine = shares + part * width;
  float sum = 0.f;
#pragma unroll 16
  for (int index = 0; index < width; ++index) sum += mine[index];
  return sum;
}

__device__ __forceinline__ float scan_join_parts(float q0, float q1, float q2, float q3, int R) {
  float sum = q0;
  if (R >= 2) sum += q1;
  if (R >= 4) sum = (sum + q2) + q3;
  return sum;
}

__device__ __forceinline__ float scan_row_sum(const float* shares, int R) {
  return scan_join_parts(scan_part_sum(shares, R, 0), R >= 2 ? scan_part_sum(shares, R, 1) : 0.f,
                         R >= 4 ? scan_part_sum(shares, R, 2) : 0.f, R >= 4 ? scan_part_sum(shares, R, 3) : 0.f, R);
}

// A barrier of the workgroup for what went through LDS, and nothing else.  __syncthreads() also waits for every load
// from memory that is under way (its fences order all memory), and the loads for the blocks ahead are meant to stay
// under way across the barriers of the block that is being scanned.
__device__ __forceinline__ void scan_lds_barrier() {
  __builtin_amdgcn_s_waitcnt(0xc07f);          // lgkmcnt(0): this wave's LDS reads and writes are done; vmcnt, expcnt: any
  __builtin_amdgcn_s_barrier();
}

// lane `which` of every group of four lanes, in all four (the data-parallel quad permutation)
template <int WHICH>
__device__ __forceinline__ float scan_quad_lane(float v) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), WHICH * 0x55, 0xf, 0xf, true));
}

// VECTORS (staged kernel only): B and C come four neighbouring elements a load (N, the row stride and the columns
// of B are multiples of 4 and the rows 16-byte aligned); else element by element.
template <typename T, int PER, bool SINGLE, bool VECTORS>
__global__ void __launch_bounds__(256, 2)          // two workgroups a compute unit at least
ssm_scan_kernel(const T* __restrict__ xbc, long xbc_ld, const T* __restrict__ dt, long dt_ld,
                const float* __restrict__ dt_bias, const float* __restrict__ A, const float* __restrict__ D,
                float* __restrict__ state, const int* __restrict__ cu_seqlens, const int* __restrict__ slot_ids,
                int H, int P, int N, int G, int R, int block_tokens, float* __restrict__ y, long y_ld) {
  constexpr int TB = PER == 1 ? SCAN_BLOCK_ELEMENTS / 2 : SCAN_BLOCK_ELEMENTS / PER;    // tokens of a block at most (block_tokens <= TB: a block's x
                                                       // values are one a thread)
  extern __shared__ __align__(16) float shares_l[];    // [tokens of a block][rows_per_block][R shares, then the row's x]
  __shared__ float decay_l[2][TB], delta_l[2][TB];
  const int lane = blockIdx.z;
  const int head = blockIdx.y;
  const int tid = threadIdx.x;
  const int rows_per_block = 256 / R;
  const int row_in_block = tid / R;
  const int r = tid - row_in_block * R;
  const int p0 = blockIdx.x * rows_per_block;
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
  const float a = A[head];
  const float bias = dt_bias[head];
  const float skip = D[head];
  // the state is waited for here, once: left to the compiler, the wait lands inside the loop over the blocks, where
  // it also waits for the loads of the blocks ahead, every time round
  __builtin_amdgcn_s_waitcnt(0x0f70);          // vmcnt(0)
  const long b_col = E + (long)group * N;
  const long c_col = E + (long)G * N + (long)group * N;
  const long x_col = (long)head * P + (active ? p : 0);
  const int share_ld = R + 1;
  const int token_ld = rows_per_block * share_ld;

  if (SINGLE) {
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
      shares_l[row_in_block * share_ld + r] = partial;
      if (r == 0) shares_l[row_in_block * share_ld + R] = x;
      __syncthreads();
      if (tid < rows_per_block && p0 + tid < P) {
        const float* shares = shares_l + tid * share_ld;
        y[t * y_ld + (long)head * P + p0 + tid] = fmaf(skip, shares[R], scan_row_sum(shares, R));
      }
      __syncthreads();
    }
  } else {
    // A block's B, C, x and dt are brought in by one of the workgroup's four waves, the waves taking turns: wave w
    // asks for the blocks w, w + 4, ... into its registers, four blocks before their turn, and lays a block in LDS
    // while the block before it is added up.  A wave's loads therefore have four blocks' time to arrive, and the
    // wait for them (which a wave can only state for all of its loads at once) never meets a load that was asked
    // for a moment ago.  Every element comes in once a workgroup: the rows of a head, and the heads of a group,
    // read the same B and C.
    float* b_l = shares_l + block_tokens * token_ld;            // [2][block_tokens][2 N]: B then C of a token
    float* x_l = b_l + 2 * block_tokens * 2 * N;                // [2][block_tokens][rows_per_block]
    typedef T pieces __attribute__((ext_vector_type(4)));
    const int row_floats = 2 * N;
    const int pieces_a_row = (row_floats + 3) / 4;
    const bool whole_rows = N == R * PER && block_tokens == TB;          // no lane of a row is idle, blocks are of TB tokens
    const int wave = tid / WAVE;
    const int lane64 = tid % WAVE;
    float staged_bc[SCAN_STAGE_PIECES][4], staged_x[4], staged_dt = 0.f;
    // where this lane's pieces lie in a block (the same for every block: worked out once, a division each)
    int piece_token[SCAN_STAGE_PIECES], piece_col[SCAN_STAGE_PIECES];
#pragma unroll
    for (int j = 0; j < SCAN_STAGE_PIECES; ++j) {
      const int index = lane64 + j * WAVE;
      piece_token[j] = index / pieces_a_row;
      piece_col[j] = (index - piece_token[j] * pieces_a_row) * 4;
    }
    const int rows_shift = __ffs(rows_per_block) - 1;               // rows_per_block is a power of two
    // block `block` of the lane into this wave's registers (nothing if the lane has no such block)
    auto fetch = [&](int block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)max(0L, min((long)block_tokens, t_end - t0));
      if (count <= 0) return;
#pragma unroll
      for (int j = 0; j < SCAN_STAGE_PIECES; ++j) {
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
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int index = min(lane64 + j * WAVE, count * rows_per_block - 1);
        const int token = index >> rows_shift;
        const int row = p0 + index - (token << rows_shift);
        staged_x[j] = row < P ? to_float(xbc[(t0 + token) * xbc_ld + (long)head * P + row]) : 0.f;
      }
      staged_dt = to_float(dt[(t0 + min(lane64, count - 1)) * dt_ld + head]);
    };
    // this wave's registers (block `block`) into LDS: B, C and x as they are, dt as delta and decay
    auto lay_down = [&](int block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)max(0L, min((long)block_tokens, t_end - t0));
      if (count <= 0) return;
      const int phase = block & 1;
      float* rows_l = b_l + phase * block_tokens * row_floats;
#pragma unroll
      for (int j = 0; j < SCAN_STAGE_PIECES; ++j) {
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
#pragma unroll
      for (int j = 0; j < 4; ++j)
        if (lane64 + j * WAVE < count * rows_per_block) x_l[phase * block_tokens * rows_per_block + lane64 + j * WAVE] = staged_x[j];
      if (lane64 < count) {
        const float delta = softplus_f(staged_dt + bias);
        delta_l[phase][lane64] = delta;
        decay_l[phase][lane64] = expf(delta * a);
      }
    };
    fetch(wave);                             // blocks 0 .. 3, one a wave
    if (wave == 0) {
      lay_down(0);
      fetch(4);
    }
    const int blocks = (int)((t_end - t_begin + block_tokens - 1) / block_tokens);
    for (int block = 0; block < blocks; ++block) {
      const long t0 = t_begin + (long)block * block_tokens;
      const int count = (int)min((long)block_tokens, t_end - t0);
      const int phase = block & 1;
      scan_lds_barrier();                   // this block's operands are laid down, and the block before has been
                                            // added up: its shares may be overwritten
      const float* rows_l = b_l + phase * block_tokens * row_floats;
      const float* x_now = x_l + phase * block_tokens * rows_per_block + row_in_block;
      const float* mine_l = rows_l + min(r * PER, N - PER > 0 ? N - PER : 0);    // this thread's columns of B (C: N further)
      float* shares_mine = shares_l + row_in_block * share_ld + r;
      // a whole block of a row whose lanes all hold PER elements runs without a condition: straight code whose
      // LDS addresses are constants; the last block of a lane and rows with idle lanes take the guarded loop
      if (count == TB && whole_rows) {
        float b[TB][PER], c[TB][PER], decay[TB], dx[TB], x[TB];
#pragma unroll
        for (int token = 0; token < TB; ++token) {
          decay[token] = decay_l[phase][token];
          x[token] = x_now[token * rows_per_block];
          dx[token] = delta_l[phase][token] * x[token];
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            b[token][i] = mine_l[token * row_floats + i];
            c[token][i] = mine_l[token * row_floats + N + i];
          }
        }
#pragma unroll
        for (int token = 0; token < TB; ++token) {
          float partial = 0.f;
#pragma unroll
          for (int i = 0; i < PER; ++i) {
            const float next_s = fmaf(decay[token], s[i], dx[token] * b[token][i]);
            s[i] = next_s;
            partial = fmaf(next_s, c[token][i], partial);
          }
          shares_mine[token * token_ld] = partial;
          if (r == 0) shares_mine[token * token_ld + R] = x[token];
        }
      } else {
        for (int token = 0; token < count; ++token) {
          const float decay = decay_l[phase][token];
          const float x = x_now[token * rows_per_block];
          const float dx = delta_l[phase][token] * x;
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
          shares_mine[token * token_ld] = partial;
          if (r == 0) shares_mine[token * token_ld + R] = x;
        }
      }
      scan_lds_barrier();
      // the wave whose turn it is lays the next block down and asks for the block four after that one
      if (wave == ((block + 1) & 3)) {
        lay_down(block + 1);
        fetch(block + 5);
      }
      // four threads an output, a quarter of the row's shares each
      const int outputs = count * rows_per_block;
      for (int first = 0; first < outputs; first += 64) {
        const int index = min(first + tid / 4, outputs - 1);
        const int token = index >> rows_shift;
        const int row = index - (token << rows_shift);
        const float* shares = shares_l + token * token_ld + row * share_ld;
        const int part = tid & 3;
        const float quarter = (part == 0 || R >= 4 || (part == 1 && R >= 2)) ? scan_part_sum(shares, R, part) : 0.f;
        const float sum = scan_join_parts(scan_quad_lane<0>(quarter), scan_quad_lane<1>(quarter), scan_quad_lane<2>(quarter),
                                          scan_quad_lane<3>(quarter), R);
        if (part == 0 && first + tid / 4 < outputs && p0 + row < P)
          y[(t0 + token) * y_ld + (long)head * P + p0 + row] = fmaf(skip, shares[R], sum);
      }
    }
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int n = r * PER + i;
      if (n < N) s_row[n] = s[i];
    }
  }
}

// longest: an upper bound of the tokens of a lane (0: unknown); a step whose lanes all hold one token takes the
// kernel without staging.
extern "C" int mi_ssm_scan(const void* xbc, int dtype, long xbc_ld, const void* dt, long dt_ld,
                           const float* dt_bias, const float* A, const float* D, float* state,
                           const int* cu_seqlens, const int* slot_ids, int num_lanes, int longest, int H, int P, int N,
                           int G, float* y, long y_ld, hipStream_t stream) {
  if (num_lanes <= 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G != 0) return ERR_BAD_ARGUMENT;
  if (N > WAVE * SCAN_MAX_PER_THREAD) return ERR_UNSUPPORTED_SIZE;
  if (H > 65535 || num_lanes > 65535) return ERR_UNSUPPORTED_SIZE;
  int R = 1;
  while (R < N && R < WAVE) R <<= 1;
  const int rows_per_block = 256 / R;
  const dim3 grid((P + rows_per_block - 1) / rows_per_block, H, num_lanes);
  const int per_needed = (N + R - 1) / R;
  const int per = per_needed <= 1 ? 1 : per_needed <= 2 ? 2 : per_needed <= 4 ? 4 : 8;
  const bool single = longest == 1;
  // tokens of a block: 16 / PER (8 at most), no more than R (so that a block's x values, one a row and token, are at most 256), and
  // B and C of a block are no more than the wave whose turn it is sends for
  int block_tokens = per == 1 ? SCAN_BLOCK_ELEMENTS / 2 : SCAN_BLOCK_ELEMENTS / per;
  if (block_tokens > R) block_tokens = R;
  while (block_tokens > 1 && (long)block_tokens * 2 * N > (long)WAVE * 4 * SCAN_STAGE_PIECES) block_tokens /= 2;
  if (single) block_tokens = 1;
  const size_t bytes = ((size_t)block_tokens * rows_per_block * (R + 1) +
                        (single ? 0 : 2 * (size_t)block_tokens * (2 * N + rows_per_block))) * sizeof(float);
  // four elements a load: every head's and group's columns of B and C start at multiples of 4
  const bool vectors = !single && N % 4 == 0 && xbc_ld % 4 == 0 && ((long)H * P) % 4 == 0 &&
                       ((uintptr_t)xbc % (dtype == DT_F32 ? 16 : 8)) == 0;
#define SCAN_LAUNCH(T_, PER_, SINGLE_, VECTORS_)                                                                     \
  ssm_scan_kernel<T_, PER_, SINGLE_, VECTORS_><<<grid, 256, bytes, stream>>>(                                        \
      (const T_*)xbc, xbc_ld, (const T_*)dt, dt_ld, dt_bias, A, D, state, cu_seqlens, slot_ids, H, P, N, G, R,       \
      block_tokens, y, y_ld)
#define SCAN_BY_PER(T_, SINGLE_, VECTORS_)                     \
  do {                                                         \
    if (per == 1) SCAN_LAUNCH(T_, 1, SINGLE_, VECTORS_);       \
    else if (per == 2) SCAN_LAUNCH(T_, 2, SINGLE_, VECTORS_);  \
    else if (per == 4) SCAN_LAUNCH(T_, 4, SINGLE_, VECTORS_);  \
    else SCAN_LAUNCH(T_, 8, SINGLE_, VECTORS_);                \
  } while (0)
#define SCAN_BY_KIND(T_)                               \
  do {                                                 \
    if (single) SCAN_BY_PER(T_, true, false);          \
    else if (vectors) SCAN_BY_PER(T_, false, true);    \
    else SCAN_BY_PER(T_, false, false);                \
  } while (0)
  if (dtype == DT_F32) SCAN_BY_KIND(float);
  else if (dtype == DT_BF16) SCAN_BY_KIND(bf16_t);
  else return ERR_BAD_ARGUMENT;
#undef SCAN_BY_KIND
#undef SCAN_BY_PER
#undef SCAN_LAUNCH
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
