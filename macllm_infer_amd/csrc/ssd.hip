// The Mamba2 selective scan for prompt portions in bfloat16, in chunks on the matrix cores
// (the "state space duality" form).  Per lane (consecutive tokens of one request), head h,
// group g of the head, with delta_t = softplus(dt_t + dt_bias), a_t = delta_t * A_h and the
// recurrence of mamba2.hip
//     S_t = exp(a_t) S_{t-1} + delta_t x_t (outer) B_t,   y_t = S_t . C_t + D_h x_t,
// cut the lane into chunks of Q tokens and let L_t be the running sum of a inside a chunk:
//     y_t   = exp(L_t) (S_in . C_t) + sum_{s<=t} exp(L_t - L_s) delta_s (C_t . B_s) x_s + D_h x_t
//     S_out = exp(L_end) S_in + sum_s exp(L_end - L_s) delta_s x_s (outer) B_s
// Every exponent is a difference of a non-increasing sequence taken forwards, so it is <= 0 and
// nothing overflows.  The result does not depend on Q beyond rounding.  Five kernels:
//     prepare     delta, L                                    (one workgroup per chunk and head)
//     transpose   x and B of each chunk, token-contiguous and zero-padded to Q: [chunk, E + G*N, Q]
//     chunk_state sum_s exp(L_end - L_s) delta_s x_s (outer) B_s  per chunk and head (matrix cores)
//     state_pass  S_in of every chunk from the slot's state, serially over a lane's chunks; the
//                 lane's final state goes back to the slot (float32 throughout)
//     chunk_scan  y: the two sums above on the matrix cores, (C . B^T) shared by the heads of a group;
//                 optionally the gate y * SiLU(z) on the way out
// Operand layouts follow attn_mfma.h: a matrix-core operand wants its contraction index
// contiguous, which is the state index n for C . B^T and S_in . C, and the token for the other
// two products, hence the transposed copies.
// (reference recurrence: crates/macllm-kernels/src/mamba2.rs:259-288; the reference scans token by token.)
#include "common.h"

typedef __bf16 s_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 s_bf16x4 __attribute__((ext_vector_type(4)));
typedef float s_floatx4 __attribute__((ext_vector_type(4)));

#define SSD_MAX_Q 256
#define SSD_HEADS_PER_BLOCK 1

// chunk table: int32 [n_chunks, 4] = (lane, first token row, length, index of the chunk within its lane)

// ---------------------------------------------------------------- prepare
// delta[t, h] = softplus(dt + bias); cum[t, h] = sum of delta*A over the chunk up to t (inclusive).
__device__ void ssd_prepare_block(const bf16_t* __restrict__ dt, long dt_ld, const float* __restrict__ dt_bias,
                                  const float* __restrict__ A, const int* __restrict__ chunks, int H,
                                  float* __restrict__ delta, float* __restrict__ cum, int chunk, int head,
                                  float* wave_total) {
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  const int s = threadIdx.x;
  const int lane = s & (WAVE - 1);
  const int wave = s / WAVE;
  float step = 0.f, a = 0.f;
  if (s < length) {
    step = softplus_f((float)dt[(long)(t0 + s) * dt_ld + head] + dt_bias[head]);
    a = step * A[head];
  }
  float running = a;                       // inclusive scan inside the wave
#pragma unroll
  for (int offset = 1; offset < WAVE; offset <<= 1) {
    const float other = __shfl_up(running, offset, WAVE);
    if (lane >= offset) running += other;
  }
  if (lane == WAVE - 1) wave_total[wave] = running;
  __syncthreads();
  float before = 0.f;
  for (int w = 0; w < wave; ++w) before += wave_total[w];
  if (s < length) {
    delta[(long)(t0 + s) * H + head] = step;
    cum[(long)(t0 + s) * H + head] = running + before;
  }
}

// ---------------------------------------------------------------- transpose
// out[chunk, channel, s] = xbc[t0 + s, channel] for s < length, 0 for the padding up to Q.
// 64 channels of a chunk per workgroup: 16-byte loads along the channels, 2-byte stores into a
// transposed LDS tile whose row stride (Q + 2 elements = an odd number of banks) keeps them
// apart, 4-byte LDS reads and 16-byte stores along the tokens.
__device__ void ssd_transpose_block(const bf16_t* __restrict__ xbc, long ld, int channels, const int* __restrict__ chunks,
                                    int Q, bf16_t* __restrict__ out, int chunk, int c0, bf16_t* tile) {
  const int stride = Q + 2;
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  for (int index = threadIdx.x; index < Q * 8; index += 256) {
    const int s = index / 8;
    const int c = (index % 8) * 8;
    s_bf16x8 v;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = (bf16_t)0.f;
    if (s < length && c0 + c < channels) v = *reinterpret_cast<const s_bf16x8*>(xbc + (long)(t0 + s) * ld + c0 + c);
#pragma unroll
    for (int j = 0; j < 8; ++j) tile[(c + j) * stride + s] = v[j];
  }
  __syncthreads();
  const int vectors = Q / 8;
  for (int index = threadIdx.x; index < 64 * vectors; index += 256) {
    const int c = index / vectors;
    const int s = (index % vectors) * 8;
    if (c0 + c >= channels) continue;
    const unsigned* words = reinterpret_cast<const unsigned*>(tile + c * stride + s);
    uint4 v;
    v.x = words[0];
    v.y = words[1];
    v.z = words[2];
    v.w = words[3];
    *reinterpret_cast<uint4*>(out + ((long)chunk * channels + c0 + c) * Q + s) = v;
  }
}

// Both in one launch (they do not depend on each other and each is too small to fill the GPU): rows
// 0 .. H-1 of the grid prepare a head, the rows after transpose 64 channels.
__global__ void __launch_bounds__(256)
ssd_prepare_transpose_kernel(const bf16_t* __restrict__ dt, long dt_ld, const float* __restrict__ dt_bias,
                             const float* __restrict__ A, const int* __restrict__ chunks, int H, float* __restrict__ delta,
                             float* __restrict__ cum, const bf16_t* __restrict__ xbc, long xbc_ld, int channels, int Q,
                             bf16_t* __restrict__ TT) {
  __shared__ __align__(4) bf16_t tile[64 * (SSD_MAX_Q + 2)];
  __shared__ float wave_total[SSD_MAX_Q / WAVE];
  if ((int)blockIdx.y < H)
    ssd_prepare_block(dt, dt_ld, dt_bias, A, chunks, H, delta, cum, blockIdx.x, blockIdx.y, wave_total);
  else
    ssd_transpose_block(xbc, xbc_ld, channels, chunks, Q, TT, blockIdx.x, ((int)blockIdx.y - H) * 64, tile);
}

// ---------------------------------------------------------------- conv, fused with the transpose
// The causal depthwise conv + SiLU of mamba2.hip (conv1d_silu) on a chunk's tokens and 64 channels, from the
// raw projection rows: the result goes to xbc[t, channel] (row-major, what the chunk scan reads for C, B and
// the skip) and, for the channels of x and B, into the transposed copy as well.  A thread takes 8 channels and
// 4 consecutive tokens; the K-1 rows before a chunk are the lane's previous tokens, or the request's conv
// tail when the chunk opens the lane.  All loads first, none under a condition (rows and channels that do
// not exist are clamped and dropped).  The tail itself is updated later, by ssd_tail_block, once every
// chunk has read it.
template <int K>
__device__ void ssd_conv_block(const bf16_t* __restrict__ u, long u_ld, int C, const float* __restrict__ conv_w,
                               const float* __restrict__ conv_b, const bf16_t* __restrict__ conv_state,
                               const int* __restrict__ chunks, const int* __restrict__ slot_ids, int Q,
                               bf16_t* __restrict__ xbc, long xbc_ld, int tt_channels, bf16_t* __restrict__ TT,
                               int chunk, int c0, bf16_t* tile) {
  constexpr int ROWS = 4;
  const int stride = Q + 2;
  const int lane_id = chunks[4 * chunk];
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  const bool opens = chunks[4 * chunk + 3] == 0;
  const bf16_t* tail = conv_state + (long)slot_ids[lane_id] * (K - 1) * C;
  const long first_row = opens ? (long)t0 : (long)t0 - (K - 1);
  const float* bias_or_taps = conv_b ? conv_b : conv_w;
  for (int item = threadIdx.x; item < (Q / ROWS) * 8; item += 256) {
    const int s0 = (item / 8) * ROWS;
    const int c = (item % 8) * 8;
    const bool real = c0 + c < C;
    const int channel = real ? c0 + c : C - 8;
    s_bf16x8 window[ROWS + K - 1], before[K - 1];
#pragma unroll
    for (int j = 0; j < ROWS + K - 1; ++j) {
      const long row = min(max((long)t0 + s0 - (K - 1) + j, first_row), (long)t0 + length - 1);
      window[j] = *reinterpret_cast<const s_bf16x8*>(u + row * u_ld + channel);
    }
#pragma unroll
    for (int j = 0; j < K - 1; ++j) before[j] = *reinterpret_cast<const s_bf16x8*>(tail + (long)j * C + channel);
    s_floatx4 taps[2 * K];                          // conv_w[channel .. channel+8, 0 .. K): 8K contiguous floats
#pragma unroll
    for (int j = 0; j < 2 * K; ++j) taps[j] = *reinterpret_cast<const s_floatx4*>(conv_w + (long)channel * K + 4 * j);
    const s_floatx4 b_lo = *reinterpret_cast<const s_floatx4*>(bias_or_taps + channel);
    const s_floatx4 b_hi = *reinterpret_cast<const s_floatx4*>(bias_or_taps + channel + 4);
    if (opens && s0 == 0) {
#pragma unroll
      for (int j = 0; j < K - 1; ++j) window[j] = before[j];
    }
    auto tap = [&](int cc, int k) { return taps[(cc * K + k) / 4][(cc * K + k) % 4]; };
#pragma unroll
    for (int i = 0; i < ROWS; ++i) {
      const int position = s0 + i;
      float sum[8];
#pragma unroll
      for (int cc = 0; cc < 8; ++cc) sum[cc] = conv_b ? (cc < 4 ? b_lo[cc] : b_hi[cc - 4]) : 0.f;
#pragma unroll
      for (int k = 0; k < K; ++k)
#pragma unroll
        for (int cc = 0; cc < 8; ++cc) sum[cc] += tap(cc, k) * (float)window[i + k][cc];
      s_bf16x8 result;
      const bool live = real && position < length;
#pragma unroll
      for (int cc = 0; cc < 8; ++cc) result[cc] = live ? (bf16_t)silu_bf16_f(sum[cc]) : (bf16_t)0.f;
      if (live) *reinterpret_cast<s_bf16x8*>(xbc + (long)(t0 + position) * xbc_ld + channel) = result;
#pragma unroll
      for (int cc = 0; cc < 8; ++cc) tile[(c + cc) * stride + position] = result[cc];
    }
  }
  __syncthreads();
  const int vectors = Q / 8;
  for (int index = threadIdx.x; index < 64 * vectors; index += 256) {
    const int c = index / vectors;
    const int position = (index % vectors) * 8;
    if (c0 + c >= tt_channels) continue;
    const unsigned* words = reinterpret_cast<const unsigned*>(tile + c * stride + position);
    uint4 v;
    v.x = words[0];
    v.y = words[1];
    v.z = words[2];
    v.w = words[3];
    *reinterpret_cast<uint4*>(TT + ((long)chunk * tt_channels + c0 + c) * Q + position) = v;
  }
}

// prepare (rows 0 .. H-1 of the grid) and the conv with the transpose (the rows after) in one launch
template <int K>
__global__ void __launch_bounds__(256)
ssd_prepare_conv_kernel(const bf16_t* __restrict__ dt, long dt_ld, const float* __restrict__ dt_bias,
                        const float* __restrict__ A, const int* __restrict__ chunks, int H, float* __restrict__ delta,
                        float* __restrict__ cum, const bf16_t* __restrict__ u, long u_ld, int C,
                        const float* __restrict__ conv_w, const float* __restrict__ conv_b,
                        const bf16_t* __restrict__ conv_state, const int* __restrict__ slot_ids, int Q,
                        bf16_t* __restrict__ xbc, long xbc_ld, int tt_channels, bf16_t* __restrict__ TT) {
  __shared__ __align__(4) bf16_t tile[64 * (SSD_MAX_Q + 2)];
  __shared__ float wave_total[SSD_MAX_Q / WAVE];
  if ((int)blockIdx.y < H)
    ssd_prepare_block(dt, dt_ld, dt_bias, A, chunks, H, delta, cum, blockIdx.x, blockIdx.y, wave_total);
  else
    ssd_conv_block<K>(u, u_ld, C, conv_w, conv_b, conv_state, chunks, slot_ids, Q, xbc, xbc_ld, tt_channels, TT,
                      blockIdx.x, ((int)blockIdx.y - H) * 64, tile);
}

// The conv tail of a lane after its tokens: the last K-1 rows of [old tail ; the lane's raw rows]
// (conv_state_update of mamba2.hip), one thread per channel; every old value is read before the first is written.
__device__ void ssd_tail_block(const bf16_t* __restrict__ u, long u_ld, int C, int K, bf16_t* __restrict__ conv_state,
                               const int* __restrict__ chunks, const int* __restrict__ lane_chunks,
                               const int* __restrict__ slot_ids, int Q, int lane, int channel) {
  if (channel >= C) return;
  const int first = lane_chunks[2 * lane];
  const int count = lane_chunks[2 * lane + 1];
  const long start = chunks[4 * first + 1];
  const long total = (long)(count - 1) * Q + chunks[4 * (first + count - 1) + 2];
  bf16_t* tail = conv_state + (long)slot_ids[lane] * (K - 1) * C + channel;
  bf16_t kept[3];
#pragma unroll
  for (int j = 0; j < 3; ++j) {
    if (j < K - 1) {
      const long source = total + j;                 // row of the (K-1 + total)-row window
      kept[j] = source < K - 1 ? tail[source * C] : u[(start + source - (K - 1)) * u_ld + channel];
    }
  }
#pragma unroll
  for (int j = 0; j < 3; ++j)
    if (j < K - 1) tail[(long)j * C] = kept[j];
}

// ---------------------------------------------------------------- chunk state
// chunk_state[chunk, h, p, n] = sum_s xT[h*P + p, s] * (BT[g*N + n, s] * exp(L_end - L_s) * delta_s)
// computed as its transpose on the matrix cores: A = weighted BT rows (n), B = xT rows (p),
// contraction over the Q tokens; a lane ends up with 4 consecutive n of one p.
// chunk_decay[chunk, h] = exp(L_end).  TT is the transposed copy [chunk, E + G*N, Q]: x rows
// first, B rows after.  QK = Q / 32 is a template parameter and a tile of rows that does not
// exist is clamped, so that all fragments of a tile are asked for at once.
template <int QK>
__global__ void __launch_bounds__(512)
ssd_chunk_state_kernel(const bf16_t* __restrict__ TT, int E, int GN, const float* __restrict__ delta,
                       const float* __restrict__ cum, const int* __restrict__ chunks, int H, int P, int N, int G,
                       float* __restrict__ chunk_state, float* __restrict__ chunk_decay) {
  constexpr int Q = 32 * QK;
  __shared__ float weight[Q];
  const int chunk = blockIdx.x;
  const int head = blockIdx.y;
  const int group = head / (H / G);
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int q = lane / 16;
  const int r = lane % 16;
  const float total = cum[(long)(t0 + length - 1) * H + head];
  for (int s = tid; s < Q; s += 512) {
    const long at = (long)(t0 + min(s, length - 1)) * H + head;
    const float value = __expf(total - cum[at]) * delta[at];
    weight[s] = s < length ? value : 0.f;
  }
  if (tid == 0) chunk_decay[(long)chunk * H + head] = __expf(total);
  __syncthreads();
  const bf16_t* x_rows = TT + ((long)chunk * (E + GN) + (long)head * P) * Q;
  const bf16_t* b_rows = TT + ((long)chunk * (E + GN) + E + (long)group * N) * Q;
  float* out = chunk_state + ((long)chunk * H + head) * P * N;
  const int p_tiles = P / 16;
  for (int nt = wave; nt < N / 16; nt += 8) {
    for (int pt0 = 0; pt0 < p_tiles; pt0 += 4) {            // four p-tiles share the weighted B fragments
      s_bf16x8 b_raw[QK], x[4][QK];
#pragma unroll
      for (int ks = 0; ks < QK; ++ks)
        b_raw[ks] = *reinterpret_cast<const s_bf16x8*>(b_rows + (long)(nt * 16 + r) * Q + 32 * ks + 8 * q);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int pt = min(pt0 + i, p_tiles - 1);
#pragma unroll
        for (int ks = 0; ks < QK; ++ks)
          x[i][ks] = *reinterpret_cast<const s_bf16x8*>(x_rows + (long)(pt * 16 + r) * Q + 32 * ks + 8 * q);
      }
      s_floatx4 acc[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] = s_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int ks = 0; ks < QK; ++ks) {
        s_bf16x8 a;
#pragma unroll
        for (int j = 0; j < 8; ++j) a[j] = (bf16_t)((float)b_raw[ks][j] * weight[32 * ks + 8 * q + j]);
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, x[i][ks], acc[i], 0, 0, 0);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
        if (pt0 + i < p_tiles)
          *reinterpret_cast<s_floatx4*>(out + (long)((pt0 + i) * 16 + r) * N + nt * 16 + 4 * q) = acc[i];
    }
  }
}

// ---------------------------------------------------------------- state pass
// Per lane, serially over its chunks: state_in[chunk] = running (rounded to bfloat16: it is a
// matrix-core operand); running = decay[chunk] * running + chunk_state[chunk].  The running state
// starts from the request's slot and goes back to it, in float32.
__global__ void ssd_state_pass_kernel(const float* __restrict__ chunk_state, const float* __restrict__ chunk_decay,
                                      const int* __restrict__ lane_chunks, const int* __restrict__ slot_ids, int H,
                                      long per_head, float* __restrict__ ssm_state, bf16_t* __restrict__ state_in,
                                      const bf16_t* __restrict__ u, long u_ld, int C, int K,
                                      bf16_t* __restrict__ conv_state, const int* __restrict__ chunks, int Q) {
  const int lane = blockIdx.z;
  if ((int)blockIdx.y >= H) {                // rows past the heads (when the conv ran here): the lane's conv tail
    if (blockIdx.x == 0)
      ssd_tail_block(u, u_ld, C, K, conv_state, chunks, lane_chunks, slot_ids, Q, lane,
                     ((int)blockIdx.y - H) * blockDim.x + threadIdx.x);
    return;
  }
  const int head = blockIdx.y;
  const long element = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (element >= per_head) return;
  const int first = lane_chunks[2 * lane];
  const int count = lane_chunks[2 * lane + 1];
  float* slot = ssm_state + ((long)slot_ids[lane] * H + head) * per_head + element;
  float running = *slot;
  constexpr int AT_ONCE = 16;                               // chunks whose loads are asked for at once, then the recurrence
  for (int c0 = first; c0 < first + count; c0 += AT_ONCE) { // (a portion of 2,048 tokens in chunks of 128: one round)
    float added[AT_ONCE], decay[AT_ONCE];
#pragma unroll
    for (int j = 0; j < AT_ONCE; ++j) {
      const int c = min(c0 + j, first + count - 1);
      added[j] = chunk_state[((long)c * H + head) * per_head + element];
      decay[j] = chunk_decay[(long)c * H + head];
    }
#pragma unroll
    for (int j = 0; j < AT_ONCE; ++j) {
      if (c0 + j < first + count) {
        state_in[((long)(c0 + j) * H + head) * per_head + element] = (bf16_t)running;
        running = decay[j] * running + added[j];
      }
    }
  }
  *slot = running;
}

// ---------------------------------------------------------------- chunk scan
// One workgroup per (chunk, group, up to HB heads of the group, 64 tokens); each of its waves
// takes a tile of 16 tokens t.  For a tile, with lane (q, n) holding column t = tile*16 + n:
//   inter:  O^T[p, t] = S_in[p, :] . C[t, :]         A = S_in rows (bfloat16), B = C rows; then * exp(L_t)
//   intra:  for 32 tokens s at a time, W^T[s, t] = B[s, :] . C[t, :] (shared by the heads), then per
//           head  P^T[s, t] = W^T exp(L_t - L_s) delta_s [s <= t]  and  O^T += xT[p, s] . P^T[s, t]
//   y[t, p] = O^T[p, t] + D x[t, p];  with z given, gated[t, p] = y * SiLU(z[t, p]) is written instead.
// 64 state rows p (4 tiles of 16) are held at a time; a larger head repeats the pass.  NK = N / 32
// is a template parameter and no load stands under a condition (a head or a tile of rows that
// does not exist is clamped to the last that does, computed and not stored): loads come back in
// order and a condition between them would make each wait for the one before.
template <int HB, int NK>
__global__ void __launch_bounds__(256)
ssd_chunk_scan_kernel(const bf16_t* __restrict__ xbc, long xbc_ld, const bf16_t* __restrict__ TT, int E,
                      const bf16_t* __restrict__ state_in, const float* __restrict__ delta,
                      const float* __restrict__ cum, const float* __restrict__ D, const int* __restrict__ chunks,
                      int Q, int H, int P, int G, float* __restrict__ y, long y_ld,
                      const bf16_t* __restrict__ z, long z_ld, bf16_t* __restrict__ gated, long gated_ld) {
  constexpr int PT = 4;
  constexpr int N = 32 * NK;
  __shared__ float L[HB][SSD_MAX_Q];
  __shared__ float step[HB][SSD_MAX_Q];
  const int chunk = blockIdx.x;
  const int heads_per_group = H / G;
  const int subsets = (heads_per_group + HB - 1) / HB;
  const int group = blockIdx.y / subsets;
  const int head0 = group * heads_per_group + (blockIdx.y % subsets) * HB;
  const int heads = min(HB, group * heads_per_group + heads_per_group - head0);
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int tile = (gridDim.z - 1 - blockIdx.z) * 4 + wave;    // the tiles with the most tokens before them first
  if ((tile - wave) * 16 >= length) return;                      // the whole workgroup
  const int q = lane / 16;
  const int n = lane % 16;
  const int end_s = min(length, (tile - wave) * 16 + 64);        // tokens any wave of the workgroup looks at
  for (int index = tid; index < HB * end_s; index += 256) {
    const int hb = index / end_s;
    const int s = index % end_s;
    const int head = head0 + min(hb, heads - 1);
    L[hb][s] = cum[(long)(t0 + s) * H + head];
    step[hb][s] = delta[(long)(t0 + s) * H + head];
  }
  __syncthreads();
  if (tile * 16 >= length) return;
  const int b_col = E + group * N;                 // columns of B and C in a row of xbc
  const int c_col = E + G * N + group * N;
  const int last_row = t0 + length - 1;
  const int t = tile * 16 + n;                     // this lane's column
  const bool has_t = t < length;
  const int t_safe = min(t, length - 1);
  const long t_row = t0 + t_safe;
  const int p_tiles = P / 16;
  // C of the column, all of N: the B operand of both score products
  s_bf16x8 c_frag[NK];
#pragma unroll
  for (int kk = 0; kk < NK; ++kk)
    c_frag[kk] = *reinterpret_cast<const s_bf16x8*>(xbc + t_row * xbc_ld + c_col + 32 * kk + 8 * q);
  if (!has_t) {
#pragma unroll
    for (int kk = 0; kk < NK; ++kk)
#pragma unroll
      for (int j = 0; j < 8; ++j) c_frag[kk][j] = (bf16_t)0.f;
  }
  for (int pt0 = 0; pt0 < p_tiles; pt0 += PT) {
    s_floatx4 acc[HB][PT];
    // inter-chunk term
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      const int head = head0 + min(hb, heads - 1);
      const float carry = __expf(L[hb][t_safe]);
#pragma unroll
      for (int pi = 0; pi < PT; ++pi) {
        const int pt = min(pt0 + pi, p_tiles - 1);
        const bf16_t* s_rows = state_in + (((long)chunk * H + head) * P + pt * 16 + n) * N + 8 * q;
        s_floatx4 sum = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
          const s_bf16x8 a = *reinterpret_cast<const s_bf16x8*>(s_rows + 32 * kk);
          sum = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, c_frag[kk], sum, 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[hb][pi][i] = sum[i] * carry;
      }
    }
    // intra-chunk term
    for (int s0 = 0; s0 <= tile * 16 + 15 && s0 < length; s0 += 32) {
      s_floatx4 w[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        w[half] = s_floatx4{0.f, 0.f, 0.f, 0.f};
        const long s_row = min((long)t0 + s0 + 16 * half + n, (long)last_row);
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
          const s_bf16x8 a = *reinterpret_cast<const s_bf16x8*>(xbc + s_row * xbc_ld + b_col + 32 * kk + 8 * q);
          w[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, c_frag[kk], w[half], 0, 0, 0);
        }
      }
      // the A operands of all heads and row tiles of this step: asked for before the exponentials
      s_bf16x4 x_lo[HB][PT], x_hi[HB][PT];
#pragma unroll
      for (int hb = 0; hb < HB; ++hb) {
        const int head = head0 + min(hb, heads - 1);
#pragma unroll
        for (int pi = 0; pi < PT; ++pi) {
          const int pt = min(pt0 + pi, p_tiles - 1);
          const bf16_t* x_row = TT + ((long)chunk * (E + G * N) + (long)head * P + pt * 16 + n) * Q + s0 + 4 * q;
          x_lo[hb][pi] = *reinterpret_cast<const s_bf16x4*>(x_row);
          x_hi[hb][pi] = *reinterpret_cast<const s_bf16x4*>(x_row + 16);
        }
      }
#pragma unroll
      for (int hb = 0; hb < HB; ++hb) {
        s_bf16x8 p_frag;
        const float l_t = L[hb][t_safe];
#pragma unroll
        for (int half = 0; half < 2; ++half)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int s = s0 + 16 * half + 4 * q + i;
            const int s_safe = min(s, length - 1);
            const bool visible = has_t && s <= t && s < length;
            const float value = visible ? w[half][i] * __expf(l_t - L[hb][s_safe]) * step[hb][s_safe] : 0.f;
            p_frag[4 * half + i] = (bf16_t)value;
          }
#pragma unroll
        for (int pi = 0; pi < PT; ++pi) {
          s_bf16x8 a;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            a[j] = x_lo[hb][pi][j];
            a[4 + j] = x_hi[hb][pi][j];
          }
          acc[hb][pi] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p_frag, acc[hb][pi], 0, 0, 0);
        }
      }
    }
    // y[t, h*P + 16 pt + 4q + i] = acc + D x: the skip and gate operands first, then the stores
    s_bf16x4 x_skip[HB][PT], gate[HB][PT];
#pragma unroll
    for (int hb = 0; hb < HB; ++hb)
#pragma unroll
      for (int pi = 0; pi < PT; ++pi) {
        const long column = (long)(head0 + min(hb, heads - 1)) * P + min(pt0 + pi, p_tiles - 1) * 16 + 4 * q;
        x_skip[hb][pi] = *reinterpret_cast<const s_bf16x4*>(xbc + t_row * xbc_ld + column);
        gate[hb][pi] = *reinterpret_cast<const s_bf16x4*>((z != nullptr ? z + t_row * z_ld : xbc + t_row * xbc_ld) + column);
      }
#pragma unroll
    for (int hb = 0; hb < HB; ++hb) {
      const float skip = D[head0 + min(hb, heads - 1)];
#pragma unroll
      for (int pi = 0; pi < PT; ++pi) {
        if (!has_t || hb >= heads || pt0 + pi >= p_tiles) continue;
        const long column = (long)(head0 + hb) * P + (pt0 + pi) * 16 + 4 * q;
        s_floatx4 out;
#pragma unroll
        for (int i = 0; i < 4; ++i) out[i] = acc[hb][pi][i] + skip * (float)x_skip[hb][pi][i];
        if (z != nullptr) {
          s_bf16x4 packed;
#pragma unroll
          for (int i = 0; i < 4; ++i) packed[i] = (bf16_t)(out[i] * silu_bf16_f((float)gate[hb][pi][i]));
          *reinterpret_cast<s_bf16x4*>(gated + t_row * gated_ld + column) = packed;
        } else {
          *reinterpret_cast<s_floatx4*>(y + t_row * y_ld + column) = out;
        }
      }
    }
  }
}

// The same with the operands that the eight tiles of 128 tokens share staged in LDS: one
// workgroup of eight waves per (chunk, head, 128 tokens), a tile of 16 tokens a wave.  S_in of
// the head (64 rows at a time), then, 64 tokens s at a time, the rows of B and the columns of
// x^T go through LDS once for all tiles instead of once per tile from the caches; only C, the
// skip and the gate are read per tile.  Rows are padded by 16 bytes so that the 16 rows a
// matrix-core operand reads fall in different banks.  Head sizes up to 128.
#define SSD_SCAN_WAVES 8
template <int NK, int PT>
__global__ void __launch_bounds__(SSD_SCAN_WAVES * WAVE)
ssd_chunk_scan_lds_kernel(const bf16_t* __restrict__ xbc, long xbc_ld, const bf16_t* __restrict__ TT, int E,
                          const bf16_t* __restrict__ state_in, const float* __restrict__ delta,
                          const float* __restrict__ cum, const float* __restrict__ D,
                          const int* __restrict__ chunks, int Q, int H, int G, float* __restrict__ y,
                          long y_ld, const bf16_t* __restrict__ z, long z_ld, bf16_t* __restrict__ gated,
                          long gated_ld) {
  constexpr int N = 32 * NK;
  constexpr int P = 16 * PT;
  constexpr int LD1 = N + 8;                     // row stride of the S / B buffer
  constexpr int LDX = 64 + 8;                    // row stride of the x^T buffer
  constexpr int THREADS = SSD_SCAN_WAVES * WAVE;
  extern __shared__ __align__(16) unsigned char scan_smem[];
  bf16_t* buf1 = reinterpret_cast<bf16_t*>(scan_smem);                 // [64][LD1]: S_in rows, then B rows
  bf16_t* buf_x = buf1 + 64 * LD1;                                     // [P][LDX]
  float* L = reinterpret_cast<float*>(buf_x + (long)P * LDX);          // [Q]
  float* step = L + Q;                                                 // [Q]
  const int chunk = blockIdx.x;
  const int head = blockIdx.y;
  const int group = head / (H / G);
  const int t0 = chunks[4 * chunk + 1];
  const int length = chunks[4 * chunk + 2];
  if (length <= 0) return;                    // a row of the table past the step's own chunks: the whole workgroup leaves
  const int part = gridDim.z - 1 - blockIdx.z;                         // the later 128 tokens first: they have more before them
  if (part * 128 >= length) return;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int q = lane / 16;
  const int n = lane % 16;
  const int tile = part * 8 + wave;
  const int end_s = min(length, part * 128 + 128);
  const int GN = G * N;
  const int b_col = E + group * N;
  const int c_col = E + GN + group * N;
  const int last_row = t0 + length - 1;
  const int t = tile * 16 + n;
  const bool tile_live = tile * 16 < length;
  const bool has_t = t < length;
  const int t_safe = min(t, length - 1);
  const long t_row = t0 + t_safe;

  for (int s = tid; s < end_s; s += THREADS) {
    L[s] = cum[(long)(t0 + s) * H + head];
    step[s] = delta[(long)(t0 + s) * H + head];
  }
  // per tile: C of the column, the skip and the gate operands (asked for now, used at the end)
  s_bf16x8 c_frag[NK];
#pragma unroll
  for (int kk = 0; kk < NK; ++kk)
    c_frag[kk] = *reinterpret_cast<const s_bf16x8*>(xbc + t_row * xbc_ld + c_col + 32 * kk + 8 * q);
  if (!has_t) {
#pragma unroll
    for (int kk = 0; kk < NK; ++kk)
#pragma unroll
      for (int j = 0; j < 8; ++j) c_frag[kk][j] = (bf16_t)0.f;
  }

  s_floatx4 acc[PT];
#pragma unroll
  for (int pi = 0; pi < PT; ++pi) acc[pi] = s_floatx4{0.f, 0.f, 0.f, 0.f};

  // ---- inter-chunk term: S_in through LDS, 64 rows at a time
  const bf16_t* s_head = state_in + ((long)chunk * H + head) * P * N;
  for (int pb = 0; pb * 64 < P; ++pb) {
    __syncthreads();
    for (int index = tid; index < 64 * (N / 8); index += THREADS) {
      const int row = index / (N / 8);
      const int v = index % (N / 8);
      const int p = min(pb * 64 + row, P - 1);
      *reinterpret_cast<s_bf16x8*>(buf1 + row * LD1 + 8 * v) =
          *reinterpret_cast<const s_bf16x8*>(s_head + (long)p * N + 8 * v);
    }
    __syncthreads();
    if (tile_live) {
#pragma unroll
      for (int pi = 0; pi < PT; ++pi) {
        if (pi / 4 == pb) {
#pragma unroll
          for (int kk = 0; kk < NK; ++kk) {
            const s_bf16x8 a = *reinterpret_cast<const s_bf16x8*>(buf1 + ((pi % 4) * 16 + n) * LD1 + 32 * kk + 8 * q);
            acc[pi] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, c_frag[kk], acc[pi], 0, 0, 0);
          }
        }
      }
    }
  }
  {
    const float carry = __expf(L[min(t_safe, end_s - 1)]);
#pragma unroll
    for (int pi = 0; pi < PT; ++pi)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[pi][i] *= carry;
  }

  // ---- intra-chunk term: 64 tokens s at a time, B rows and x^T columns through LDS
  const bf16_t* x_head = TT + ((long)chunk * (E + GN) + (long)head * P) * Q;
  for (int sb = 0; sb * 64 < end_s; ++sb) {
    __syncthreads();
    for (int index = tid; index < 64 * (N / 8); index += THREADS) {
      const int row = index / (N / 8);
      const int v = index % (N / 8);
      const long s_row = min((long)t0 + sb * 64 + row, (long)last_row);
      *reinterpret_cast<s_bf16x8*>(buf1 + row * LD1 + 8 * v) =
          *reinterpret_cast<const s_bf16x8*>(xbc + s_row * xbc_ld + b_col + 8 * v);
    }
    for (int index = tid; index < P * 8; index += THREADS) {
      const int row = index / 8;
      const int v = index % 8;
      s_bf16x8 value;
#pragma unroll
      for (int j = 0; j < 8; ++j) value[j] = (bf16_t)0.f;
      if (sb * 64 + 8 * v < Q) value = *reinterpret_cast<const s_bf16x8*>(x_head + (long)row * Q + sb * 64 + 8 * v);
      *reinterpret_cast<s_bf16x8*>(buf_x + row * LDX + 8 * v) = value;
    }
    __syncthreads();
    if (!tile_live) continue;
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int s0 = sb * 64 + 32 * j;
      if (s0 > tile * 16 + 15 || s0 >= length) continue;
      s_floatx4 w[2];
#pragma unroll
      for (int half = 0; half < 2; ++half) {
        w[half] = s_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < NK; ++kk) {
          const s_bf16x8 a = *reinterpret_cast<const s_bf16x8*>(buf1 + (32 * j + 16 * half + n) * LD1 + 32 * kk + 8 * q);
          w[half] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, c_frag[kk], w[half], 0, 0, 0);
        }
      }
      s_bf16x8 p_frag;
      const float l_t = L[min(t_safe, end_s - 1)];
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int s = s0 + 16 * half + 4 * q + i;
          const int s_safe = min(s, end_s - 1);
          const bool visible = has_t && s <= t && s < length;
          const float value = visible ? w[half][i] * __expf(l_t - L[s_safe]) * step[s_safe] : 0.f;
          p_frag[4 * half + i] = (bf16_t)value;
        }
#pragma unroll
      for (int pi = 0; pi < PT; ++pi) {
        const bf16_t* x_row = buf_x + (pi * 16 + n) * LDX + 32 * j + 4 * q;
        const s_bf16x4 lo = *reinterpret_cast<const s_bf16x4*>(x_row);
        const s_bf16x4 hi = *reinterpret_cast<const s_bf16x4*>(x_row + 16);
        s_bf16x8 a;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          a[e] = lo[e];
          a[4 + e] = hi[e];
        }
        acc[pi] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, p_frag, acc[pi], 0, 0, 0);
      }
    }
  }

  // ---- y[t, h*P + 16 pi + 4q + i] = acc + D x
  if (!has_t) return;
  const float skip = D[head];
  s_bf16x4 x_skip[PT], gate[PT];
#pragma unroll
  for (int pi = 0; pi < PT; ++pi) {
    const long column = (long)head * P + pi * 16 + 4 * q;
    x_skip[pi] = *reinterpret_cast<const s_bf16x4*>(xbc + t_row * xbc_ld + column);
    gate[pi] = *reinterpret_cast<const s_bf16x4*>((z != nullptr ? z + t_row * z_ld : xbc + t_row * xbc_ld) + column);
  }
#pragma unroll
  for (int pi = 0; pi < PT; ++pi) {
    const long column = (long)head * P + pi * 16 + 4 * q;
    s_floatx4 out;
#pragma unroll
    for (int i = 0; i < 4; ++i) out[i] = acc[pi][i] + skip * (float)x_skip[pi][i];
    if (z != nullptr) {
      s_bf16x4 packed;
#pragma unroll
      for (int i = 0; i < 4; ++i) packed[i] = (bf16_t)(out[i] * silu_bf16_f((float)gate[pi][i]));
      *reinterpret_cast<s_bf16x4*>(gated + t_row * gated_ld + column) = packed;
    } else {
      *reinterpret_cast<s_floatx4*>(y + t_row * y_ld + column) = out;
    }
  }
}

static size_t ssd_scan_lds_bytes(int Q, int P, int N) {
  return (size_t)64 * (N + 8) * 2 + (size_t)P * (64 + 8) * 2 + (size_t)2 * Q * 4;
}

// Sizes: bfloat16; Q a multiple of 32 and at most 256; head_dim P a multiple of 16; state size N a
// multiple of 32 and at most 256; row strides multiples of 8 elements.  Otherwise
// ERR_UNSUPPORTED_SIZE (the caller uses mi_ssm_scan).
extern "C" int mi_ssd_supported(int Q, int P, int N, int G, int E) {
  return (Q % 32 == 0 && Q > 0 && Q <= SSD_MAX_Q && P % 16 == 0 && N % 32 == 0 && N <= 256 &&
          (E % 8) == 0 && ((long)G * N) % 8 == 0) ? 1 : 0;
}

extern "C" int mi_ssd_prefill(const void* xbc, long xbc_ld, const void* dt, long dt_ld, const float* dt_bias,
                              const float* A, const float* D, float* ssm_state, const int* chunks, int n_chunks,
                              const int* lane_chunks, const int* slot_ids, int n_lanes, int Q, int H, int P, int N,
                              int G, float* delta, float* cum, void* TT, float* chunk_state,
                              float* chunk_decay, void* state_in, float* y, long y_ld, const void* z, long z_ld,
                              void* gated, long gated_ld, const void* u, long u_ld, const float* conv_w,
                              const float* conv_b, void* conv_state, int conv_k, hipStream_t stream) {
  if (n_chunks <= 0 || n_lanes <= 0 || H <= 0 || G <= 0 || H % G != 0) return ERR_BAD_ARGUMENT;
  const int E = H * P;
  const int GN = G * N;
  const int C = E + 2 * GN;
  const bool conv_here = u != nullptr;       // xbc is then written here, from the raw rows u [T, C] (+ u_ld)
  if (conv_here && (!conv_w || !conv_state || conv_k < 2 || conv_k > 4 || u_ld % 8 != 0 || C % 8 != 0 ||
                    ((uintptr_t)u % 16) != 0 || ((uintptr_t)conv_state % 16) != 0 || ((uintptr_t)conv_w % 16) != 0 ||
                    ((uintptr_t)conv_b % 16) != 0 || H + (C + 63) / 64 > 65535 || H + (C + 255) / 256 > 65535))
    return ERR_UNSUPPORTED_SIZE;
  if ((z == nullptr) != (gated == nullptr) || (z == nullptr && y == nullptr)) return ERR_BAD_ARGUMENT;
  if (!mi_ssd_supported(Q, P, N, G, E) || xbc_ld % 8 != 0 || y_ld % 4 != 0 || z_ld % 4 != 0 || gated_ld % 4 != 0 ||
      n_chunks > 65535 * 32 ||
      H + (E + GN + 63) / 64 > 65535 || n_lanes > 65535)
    return ERR_UNSUPPORTED_SIZE;
  if (conv_here) {
    const dim3 grid(n_chunks, H + (C + 63) / 64);
#define CONV_CASE(K_)                                                                                              \
  ssd_prepare_conv_kernel<K_><<<grid, 256, 0, stream>>>((const bf16_t*)dt, dt_ld, dt_bias, A, chunks, H, delta, cum,  \
                                                        (const bf16_t*)u, u_ld, C, conv_w, conv_b,                  \
                                                        (const bf16_t*)conv_state, slot_ids, Q, (bf16_t*)xbc,       \
                                                        xbc_ld, E + GN, (bf16_t*)TT)
    if (conv_k == 2) CONV_CASE(2);
    else if (conv_k == 3) CONV_CASE(3);
    else CONV_CASE(4);
#undef CONV_CASE
    RETURN_IF_LAUNCH_FAILED();
  } else {
    const dim3 grid(n_chunks, H + (E + GN + 63) / 64);       // x and B are neighbours in a row of xbc
    ssd_prepare_transpose_kernel<<<grid, 256, 0, stream>>>((const bf16_t*)dt, dt_ld, dt_bias, A, chunks, H, delta, cum,
                                                           (const bf16_t*)xbc, xbc_ld, E + GN, Q, (bf16_t*)TT);
    RETURN_IF_LAUNCH_FAILED();
  }
  {
    const dim3 grid(n_chunks, H);
#define STATE_CASE(QK_)                                                                                         \
  case QK_:                                                                                                     \
    ssd_chunk_state_kernel<QK_><<<grid, 512, 0, stream>>>((const bf16_t*)TT, E, GN, delta, cum, chunks, H, P, N, G, \
                                                          chunk_state, chunk_decay);                          \
    break;
    switch (Q / 32) {
      STATE_CASE(1) STATE_CASE(2) STATE_CASE(3) STATE_CASE(4) STATE_CASE(5) STATE_CASE(6) STATE_CASE(7) STATE_CASE(8)
      default: return ERR_UNSUPPORTED_SIZE;
    }
#undef STATE_CASE
    RETURN_IF_LAUNCH_FAILED();
  }
  {
    const long per_head = (long)P * N;
    const dim3 grid((unsigned)((per_head + 255) / 256), H + (conv_here ? (C + 255) / 256 : 0), n_lanes);
    ssd_state_pass_kernel<<<grid, 256, 0, stream>>>(chunk_state, chunk_decay, lane_chunks, slot_ids, H, per_head,
                                                    ssm_state, (bf16_t*)state_in, (const bf16_t*)u, u_ld, C, conv_k,
                                                    (bf16_t*)conv_state, chunks, Q);
    RETURN_IF_LAUNCH_FAILED();
  }
  const bool staged = (P == 16 || P == 32 || P == 64 || P == 128) && (N == 32 || N == 64 || N == 128 || N == 256) &&
                      ssd_scan_lds_bytes(Q, P, N) <= 64 * 1024;
  if (staged) {
    const dim3 grid(n_chunks, H, (Q + 127) / 128);
    const size_t lds = ssd_scan_lds_bytes(Q, P, N);
#define SCAN_LDS_CASE(NK_, PT_)                                                                                   \
  if (N == 32 * NK_ && P == 16 * PT_)                                                                             \
    ssd_chunk_scan_lds_kernel<NK_, PT_><<<grid, SSD_SCAN_WAVES * WAVE, lds, stream>>>(                            \
        (const bf16_t*)xbc, xbc_ld, (const bf16_t*)TT, E, (const bf16_t*)state_in, delta, cum, D, chunks, Q, H, G, \
        y, y_ld, (const bf16_t*)z, z_ld, (bf16_t*)gated, gated_ld);
    SCAN_LDS_CASE(1, 1) SCAN_LDS_CASE(1, 2) SCAN_LDS_CASE(1, 4) SCAN_LDS_CASE(1, 8)
    SCAN_LDS_CASE(2, 1) SCAN_LDS_CASE(2, 2) SCAN_LDS_CASE(2, 4) SCAN_LDS_CASE(2, 8)
    SCAN_LDS_CASE(4, 1) SCAN_LDS_CASE(4, 2) SCAN_LDS_CASE(4, 4) SCAN_LDS_CASE(4, 8)
    SCAN_LDS_CASE(8, 1) SCAN_LDS_CASE(8, 2) SCAN_LDS_CASE(8, 4) SCAN_LDS_CASE(8, 8)
#undef SCAN_LDS_CASE
    RETURN_IF_LAUNCH_FAILED();
  } else {
    const int subsets = (H / G + SSD_HEADS_PER_BLOCK - 1) / SSD_HEADS_PER_BLOCK;
    const dim3 grid(n_chunks, G * subsets, (Q + 63) / 64);
#define SCAN_CASE(NK_)                                                                                            \
  case NK_:                                                                                                       \
    ssd_chunk_scan_kernel<SSD_HEADS_PER_BLOCK, NK_><<<grid, 256, 0, stream>>>(                                    \
        (const bf16_t*)xbc, xbc_ld, (const bf16_t*)TT, E, (const bf16_t*)state_in, delta, cum, D, chunks, Q, H, P, \
        G, y, y_ld, (const bf16_t*)z, z_ld, (bf16_t*)gated, gated_ld);                                          \
    break;
    switch (N / 32) {
      SCAN_CASE(1) SCAN_CASE(2) SCAN_CASE(3) SCAN_CASE(4) SCAN_CASE(5) SCAN_CASE(6) SCAN_CASE(7) SCAN_CASE(8)
      default: return ERR_UNSUPPORTED_SIZE;
    }
#undef SCAN_CASE
    RETURN_IF_LAUNCH_FAILED();
  }
  return 0;
}
