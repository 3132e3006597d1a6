// Fused kernels for decode steps in bfloat16: every lane of the batch holds one token, the
// batch is small (M <= 64 rows), and a step is bound by weight reads and by the latency of
// each dependent kernel.  Two kernels cover a layer's hot path:
//
//   fused_gemm : out[M, N] = epilogue( prologue(x)[M, K] . W[N, K]^T + bias )
//       prologue  NORM : x = (h + delta0 + delta1) / sqrt(mean(.^2) + eps) * w   (residual add
//                        and RMSNorm; block 0 also writes the summed residual to h_out)
//                 PLAIN: x given in bfloat16
//       epilogue  PLAIN : bfloat16 or float32 (x scale) store
//                 SWIGLU: rows come in tiles of 8 gate rows + 8 up rows; stores SiLU(g)*u
//                 CONV  : rows in [conv_lo, conv_hi) are channels of a causal depthwise conv
//                         with K taps: the new sample joins the request's tail, the tail is
//                         rolled, SiLU(conv) is stored; other rows are stored as they are
//     Each block owns 16 output rows; its 4 waves split K and feed the matrix cores
//     (v_mfma_f32_16x16x32_bf16: A = 16 weight rows x 32 k, B = 16 batch rows x 32 k, both
//     contiguous in k), then sum their partial tiles through LDS.
//
//   mixer_decode : one launch with two kinds of blocks
//       attention blocks: split-context attention as in attention.hip, with the rotation of q
//         and of the new key, the write of the new K and V into their cache cell, and the merge
//         of the splits (by the last block of each (token, kv head) to finish) folded in;
//       state-space blocks: one step of the selective scan from and into the slot state, D skip
//         and the SiLU(z) gate.
//
// Formulas and their reference lines are the ones cited in common.hip, attention.hip and
// mamba2.hip; these kernels only change what runs together.
#include "common.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define FG_THREADS 256
#define FG_WAVES 4
#define FG_PAD 8

enum { PRO_NORM = 0, PRO_PLAIN = 1 };
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_CONV = 2 };

struct FusedGemmParams {
  const float* h_in;
  const bf16_t* delta0;
  const bf16_t* delta1;
  float* h_out;
  const float* norm_w;
  float eps;
  const bf16_t* x;
  long x_ld;
  const bf16_t* W;
  const float* bias;
  int M, N, K;
  void* out;
  long out_ld;
  int out_f32;
  float out_scale;
  int conv_lo, conv_hi, conv_k;
  const float* conv_w;
  const float* conv_b;
  bf16_t* conv_state;
  const int* slot_ids;
};

__device__ __forceinline__ float round_bf16(float v) { return (float)(bf16_t)v; }

template <int MT, int PRO, int EPI>
__global__ void __launch_bounds__(FG_THREADS) fused_gemm_kernel(FusedGemmParams p) {
  extern __shared__ __align__(16) unsigned char smem[];
  const int K = p.K;
  const int ldx = K + FG_PAD;
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);
  float* red = reinterpret_cast<float*>(smem + (PRO == PRO_NORM ? (size_t)MT * 16 * ldx * sizeof(bf16_t) : 0));
  float* tile = red + FG_WAVES * MT * 256;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  if (PRO == PRO_NORM) {
    // one wave per row: sum of squares in float32, then the normalized row in bfloat16
    for (int m = wave; m < MT * 16; m += FG_WAVES) {
      bf16_t* x_row = xs + (long)m * ldx;
      if (m < p.M) {
        const float* h_row = p.h_in + (long)m * K;
        const bf16_t* d0 = p.delta0 ? p.delta0 + (long)m * K : nullptr;
        const bf16_t* d1 = p.delta1 ? p.delta1 + (long)m * K : nullptr;
        float sum_squares = 0.f;
        for (int k = lane * 4; k < K; k += WAVE * 4) {
          floatx4 v = *reinterpret_cast<const floatx4*>(h_row + k);
          if (d0) {
            const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(d0 + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] += (float)d[j];
          }
          if (d1) {
            const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(d1 + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] += (float)d[j];
          }
#pragma unroll
          for (int j = 0; j < 4; ++j) sum_squares += v[j] * v[j];
        }
        sum_squares = wave_sum(sum_squares);
        const float denominator = sqrtf(sum_squares / (float)K + p.eps);
        for (int k = lane * 4; k < K; k += WAVE * 4) {
          floatx4 v = *reinterpret_cast<const floatx4*>(h_row + k);
          if (d0) {
            const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(d0 + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] += (float)d[j];
          }
          if (d1) {
            const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(d1 + k);
#pragma unroll
            for (int j = 0; j < 4; ++j) v[j] += (float)d[j];
          }
          if (blockIdx.x == 0 && p.h_out) *reinterpret_cast<floatx4*>(p.h_out + (long)m * K + k) = v;
          const floatx4 w = *reinterpret_cast<const floatx4*>(p.norm_w + k);
          bf16x4_t packed;
#pragma unroll
          for (int j = 0; j < 4; ++j) packed[j] = (bf16_t)(v[j] / denominator * w[j]);
          *reinterpret_cast<bf16x4_t*>(x_row + k) = packed;
        }
      } else {
        for (int k = lane * 4; k < K; k += WAVE * 4) {
          bf16x4_t zero = {(bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f, (bf16_t)0.f};
          *reinterpret_cast<bf16x4_t*>(x_row + k) = zero;
        }
      }
    }
    __syncthreads();
  }

  // the product: wave w takes k-chunks w, w+4, ... of 32
  const int n0 = blockIdx.x * 16;
  const int q = lane / 16;
  const int r = lane % 16;
  const int n_row = min(n0 + r, p.N - 1);
  const bf16_t* w_row = p.W + (long)n_row * K + 8 * q;
  floatx4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  const int chunks = K / 32;
  const int iterations = (chunks - wave + FG_WAVES - 1) / FG_WAVES;
#pragma unroll 4
  for (int iteration = 0; iteration < iterations; ++iteration) {
    const int c = wave + iteration * FG_WAVES;
    const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(w_row + c * 32);
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      bf16x8_t b;
      if (PRO == PRO_NORM) {
        b = *reinterpret_cast<const bf16x8_t*>(xs + (long)(mt * 16 + r) * ldx + c * 32 + 8 * q);
      } else {
        const int m = mt * 16 + r;
        if (m < p.M) {
          b = *reinterpret_cast<const bf16x8_t*>(p.x + (long)m * p.x_ld + c * 32 + 8 * q);
        } else {
#pragma unroll
          for (int j = 0; j < 8; ++j) b[j] = (bf16_t)0.f;
        }
      }
      acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[mt], 0, 0, 0);
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int i = 0; i < 4; ++i) red[(wave * MT + mt) * 256 + i * 64 + lane] = acc[mt][i];
  __syncthreads();

  for (int index = tid; index < MT * 256; index += FG_THREADS) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < FG_WAVES; ++w) v += red[w * MT * 256 + index];
    const int mt = index / 256;
    const int i = (index % 256) / 64;
    const int l = index % 64;
    const int n_local = 4 * (l / 16) + i;
    const int n = n0 + n_local;
    const int m = mt * 16 + (l % 16);
    if (p.bias && n < p.N) v += p.bias[n];
    if (EPI == EPI_SWIGLU) {
      tile[n_local * (MT * 16) + m] = v;
      continue;
    }
    if (n >= p.N || m >= p.M) continue;
    if (EPI == EPI_CONV && n >= p.conv_lo && n < p.conv_hi) {
      const int channel = n - p.conv_lo;
      const int channels = p.conv_hi - p.conv_lo;
      const int taps = p.conv_k;
      bf16_t* tail = p.conv_state + (long)p.slot_ids[m] * (taps - 1) * channels + channel;
      const bf16_t sample = (bf16_t)v;
      float sum = p.conv_b ? p.conv_b[channel] : 0.f;
      for (int k = 0; k < taps - 1; ++k) {
        const bf16_t old = tail[(long)k * channels];
        sum += p.conv_w[channel * taps + k] * (float)old;
        if (k > 0) tail[(long)(k - 1) * channels] = old;       // roll the tail by one
      }
      sum += p.conv_w[channel * taps + taps - 1] * (float)sample;
      if (taps > 1) tail[(long)(taps - 2) * channels] = sample;
      reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + n] = (bf16_t)silu_f(sum);
    } else if (p.out_f32) {
      reinterpret_cast<float*>(p.out)[(long)m * p.out_ld + n] = v * p.out_scale;
    } else {
      reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + n] = (bf16_t)(v * p.out_scale);
    }
  }
  if (EPI == EPI_SWIGLU) {
    __syncthreads();
    const int half_rows = p.N / 2;
    for (int index = tid; index < 8 * MT * 16; index += FG_THREADS) {
      const int i = index / (MT * 16);
      const int m = index % (MT * 16);
      const int column = blockIdx.x * 8 + i;
      if (m >= p.M || column >= half_rows) continue;
      const float gate = round_bf16(tile[i * (MT * 16) + m]);
      const float up = round_bf16(tile[(8 + i) * (MT * 16) + m]);
      reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + column] = (bf16_t)(silu_f(gate) * up);
    }
  }
}

static size_t fused_gemm_lds(int MT, int pro, int K) {
  size_t bytes = (size_t)FG_WAVES * MT * 256 * sizeof(float) + (size_t)16 * MT * 16 * sizeof(float);
  if (pro == PRO_NORM) bytes += (size_t)MT * 16 * (K + FG_PAD) * sizeof(bf16_t);
  return bytes;
}

template <int MT>
static int launch_fused_gemm(const FusedGemmParams& p, int pro, int epi, hipStream_t stream) {
  const int blocks = (p.N + 15) / 16;
  const size_t lds = fused_gemm_lds(MT, pro, p.K);
#define FG_LAUNCH(PRO_, EPI_) \
  fused_gemm_kernel<MT, PRO_, EPI_><<<blocks, FG_THREADS, lds, stream>>>(p)
  if (pro == PRO_NORM && epi == EPI_PLAIN) FG_LAUNCH(PRO_NORM, EPI_PLAIN);
  else if (pro == PRO_NORM && epi == EPI_SWIGLU) FG_LAUNCH(PRO_NORM, EPI_SWIGLU);
  else if (pro == PRO_NORM && epi == EPI_CONV) FG_LAUNCH(PRO_NORM, EPI_CONV);
  else if (pro == PRO_PLAIN && epi == EPI_PLAIN) FG_LAUNCH(PRO_PLAIN, EPI_PLAIN);
  else if (pro == PRO_PLAIN && epi == EPI_SWIGLU) FG_LAUNCH(PRO_PLAIN, EPI_SWIGLU);
  else if (pro == PRO_PLAIN && epi == EPI_CONV) FG_LAUNCH(PRO_PLAIN, EPI_CONV);
  else return ERR_BAD_ARGUMENT;
#undef FG_LAUNCH
  return 0;
}

// Sizes: 1 <= M <= 64, K a multiple of 32; with the NORM prologue the normalized rows must fit
// 64 KiB of LDS beside the reduction area.  EPI_SWIGLU wants N a multiple of 16.
extern "C" int mi_fused_gemm(int pro, int epi, const float* h_in, const void* delta0, const void* delta1,
                             float* h_out, const float* norm_w, float eps, const void* x, long x_ld,
                             const void* W, const float* bias, int M, int N, int K, void* out, long out_ld,
                             int out_f32, float out_scale, int conv_lo, int conv_hi, int conv_k,
                             const float* conv_w, const float* conv_b, void* conv_state, const int* slot_ids,
                             hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !out) return ERR_BAD_ARGUMENT;
  if (M > 64 || K % 32 != 0) return ERR_UNSUPPORTED_SIZE;
  if (pro == PRO_NORM && (!h_in || !norm_w || h_out == h_in)) return ERR_BAD_ARGUMENT;
  if (pro == PRO_PLAIN && (!x || x_ld < K || x_ld % 8 != 0)) return ERR_BAD_ARGUMENT;
  if (epi == EPI_SWIGLU && (N % 16 != 0 || out_f32)) return ERR_BAD_ARGUMENT;
  if (epi == EPI_CONV && (conv_lo < 0 || conv_hi > N || conv_hi <= conv_lo || conv_k < 1 || !conv_w ||
                          (conv_k > 1 && (!conv_state || !slot_ids)) || out_f32))
    return ERR_BAD_ARGUMENT;
  const int MT = (M + 15) / 16;
  if (fused_gemm_lds(MT, pro, K) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p;
  p.h_in = h_in;
  p.delta0 = (const bf16_t*)delta0;
  p.delta1 = (const bf16_t*)delta1;
  p.h_out = h_out;
  p.norm_w = norm_w;
  p.eps = eps;
  p.x = (const bf16_t*)x;
  p.x_ld = x_ld;
  p.W = (const bf16_t*)W;
  p.bias = bias;
  p.M = M;
  p.N = N;
  p.K = K;
  p.out = out;
  p.out_ld = out_ld;
  p.out_f32 = out_f32;
  p.out_scale = out_scale;
  p.conv_lo = conv_lo;
  p.conv_hi = conv_hi;
  p.conv_k = conv_k;
  p.conv_w = conv_w;
  p.conv_b = conv_b;
  p.conv_state = (bf16_t*)conv_state;
  p.slot_ids = slot_ids;
  int code;
  if (MT == 1) code = launch_fused_gemm<1>(p, pro, epi, stream);
  else if (MT == 2) code = launch_fused_gemm<2>(p, pro, epi, stream);
  else if (MT == 3) code = launch_fused_gemm<3>(p, pro, epi, stream);
  else code = launch_fused_gemm<4>(p, pro, epi, stream);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// Whether mi_fused_gemm covers a shape (the host asks before it builds a fused path).
extern "C" int mi_fused_gemm_supported(int pro, int M, int K) {
  if (M <= 0 || M > 64 || K % 32 != 0) return 0;
  return fused_gemm_lds((M + 15) / 16, pro, K) <= 64 * 1024 ? 1 : 0;
}

// ---------------------------------------------------------------- mixer decode
#define MX_THREADS 256
#define MX_WAVES 4
#define MX_MAX_SPLIT 512
#define MX_SCAN_PER_THREAD 8

struct MixerParams {
  // the layer's projected row per token: [q | k | v | z | x B C (after conv) | dt], bfloat16
  const bf16_t* u;
  long u_ld;
  int M;
  // attention
  int Hq, Hkv, q_col, k_col, v_col;
  const float* inv_freq;
  int rotary_dim;
  bf16_t* k_base;
  bf16_t* v_base;
  long page_stride;
  int page_size;
  const int* block_tables;
  int max_pages;
  const int* positions;
  const int* slot_mapping;
  float scale;
  int window, split_keys, splits;
  float* partial_o;
  float* partial_ml;
  int* counters;
  // state space
  int H, P, N, G, R, p_tiles, z_col, x_col, dt_col;
  const float* dt_bias;
  const float* A;
  const float* D;
  float* ssm_state;
  const int* slot_ids;
  // outputs
  bf16_t* attn_out;       // [M, out_ld] at attn_out; attention heads first
  bf16_t* ssm_out;        // gated y, bfloat16 (when no norm follows)
  float* ssm_y;           // or float32 y before the gate (when a grouped norm follows)
  long out_ld;
  int attention_blocks;
};

// one dim of a rotated head: pairs (j, j + rotary_dim/2) of the first rotary_dim dims
__device__ __forceinline__ float rotated_dim(const bf16_t* head, int dim, int rotary_dim, float position,
                                             const float* inv_freq) {
  const float x = (float)head[dim];
  if (dim >= rotary_dim) return x;
  const int half = rotary_dim / 2;
  const int j = dim < half ? dim : dim - half;
  const float angle = position * inv_freq[j];
  const float s = sinf(angle), c = cosf(angle);
  return dim < half ? x * c - (float)head[dim + half] * s : x * c + (float)head[dim - half] * s;
}

template <int DH, int G>
__device__ void mixer_attention_block(const MixerParams& p, int block, float (*s_lds)[MX_MAX_SPLIT],
                                      float (*red)[8], float* acc_lds, int* flag) {
  constexpr int LPR = DH / 8;
  constexpr int KPW = WAVE / LPR;
  constexpr int KPB = KPW * MX_WAVES;
  constexpr int DPL = DH / WAVE;
  const int split = block % p.splits;
  const int kvh = (block / p.splits) % p.Hkv;
  const long token = block / (p.splits * p.Hkv);
  const int pos = p.positions[token];
  int first_key = 0;
  if (p.window > 0 && pos - p.window + 1 > 0) first_key = pos - p.window + 1;
  const int first_page_key = (first_key / p.page_size) * p.page_size;
  const int range_lo = first_page_key + split * p.split_keys;
  if (range_lo > pos) return;
  const int range_hi = min(range_lo + p.split_keys, pos + 1);
  const int count = range_hi - range_lo;
  const int used = min(p.splits, (pos - first_page_key) / p.split_keys + 1);
  const int* table = p.block_tables + token * p.max_pages;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int r = lane / LPR;
  const int c = lane % LPR;
  const bf16_t* row = p.u + token * p.u_ld;
  const float position = (float)pos;

  // the block whose range ends at the new token writes its rotated key and its value first
  if (range_hi == pos + 1) {
    const long cell = p.slot_mapping[token];
    const long page = cell / p.page_size;
    const int offset = (int)(cell - page * p.page_size);
    for (int dim = tid; dim < DH; dim += MX_THREADS) {
      const float k = p.inv_freq ? rotated_dim(row + p.k_col + kvh * DH, dim, p.rotary_dim, position, p.inv_freq)
                                 : (float)row[p.k_col + kvh * DH + dim];
      p.k_base[page * p.page_stride + ((long)kvh * p.page_size + offset) * DH + dim] = (bf16_t)k;
      p.v_base[page * p.page_stride + ((long)kvh * DH + dim) * p.page_size + offset] = row[p.v_col + kvh * DH + dim];
    }
    __threadfence_block();
    __syncthreads();
  }

  float qf[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const bf16_t* head = row + p.q_col + (kvh * G + g) * DH;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int dim = c * 8 + j;
      const float value = p.inv_freq ? rotated_dim(head, dim, p.rotary_dim, position, p.inv_freq) : (float)head[dim];
      qf[g][j] = round_bf16(value) * p.scale;      // q is rounded to bfloat16 after rotation, as when it is stored
    }
  }

  for (int base = 0; base < count; base += KPB) {
    const int local = base + wave * KPW + r;
    const int key = range_lo + local;
    const bool valid = local < count;
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) s[g] = 0.f;
    if (valid) {
      const int page = table[key / p.page_size];
      const int offset = key % p.page_size;
      const bf16x8_t packed = *reinterpret_cast<const bf16x8_t*>(
          p.k_base + (long)page * p.page_stride + ((long)kvh * p.page_size + offset) * DH + c * 8);
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) s[g] = fmaf(qf[g][j], (float)packed[j], s[g]);
    }
#pragma unroll
    for (int offset = LPR / 2; offset > 0; offset >>= 1)
#pragma unroll
      for (int g = 0; g < G; ++g) s[g] += __shfl_xor(s[g], offset, WAVE);
    if (valid && c == 0) {
#pragma unroll
      for (int g = 0; g < G; ++g) s_lds[g][local] = key >= first_key ? s[g] : -INFINITY;
    }
  }
  __syncthreads();

  float m[G], l[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = -INFINITY;
    for (int i = tid; i < count; i += MX_THREADS) v = fmaxf(v, s_lds[g][i]);
    v = wave_max(v);
    if (lane == 0) red[wave][g] = v;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = red[0][g];
#pragma unroll
    for (int w = 1; w < MX_WAVES; ++w) v = fmaxf(v, red[w][g]);
    m[g] = v;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float sum = 0.f;
    for (int i = tid; i < count; i += MX_THREADS) {
      const float e = __expf(s_lds[g][i] - m[g]);
      s_lds[g][i] = e;
      sum += e;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave][g] = sum;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < MX_WAVES; ++w) v += red[w][g];
    l[g] = v;
  }

  float acc[G][DPL];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[g][i] = 0.f;
  const int range_pages = (count + p.page_size - 1) / p.page_size;
  for (int pg = wave; pg < range_pages; pg += MX_WAVES) {
    const int local0 = pg * p.page_size;
    const int page = table[(range_lo + local0) / p.page_size];
    const int keys_here = min(p.page_size, count - local0);
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int dim = lane + i * WAVE;
      const bf16_t* v_row = p.v_base + (long)page * p.page_stride + ((long)kvh * DH + dim) * p.page_size;
      for (int j0 = 0; j0 < keys_here; j0 += 8) {
        const bf16x8_t packed = *reinterpret_cast<const bf16x8_t*>(v_row + j0);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (j0 + j < keys_here) {
            const float value = (float)packed[j];
#pragma unroll
            for (int g = 0; g < G; ++g) acc[g][i] = fmaf(s_lds[g][local0 + j0 + j], value, acc[g][i]);
          }
        }
      }
    }
  }
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc_lds[(wave * G + g) * DH + lane + i * WAVE] = acc[g][i];
  __syncthreads();
  const long head0 = token * p.Hq + kvh * G;
  for (int index = tid; index < G * DH; index += MX_THREADS) {
    const int g = index / DH;
    const int dim = index - g * DH;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < MX_WAVES; ++w) sum += acc_lds[(w * G + g) * DH + dim];
    p.partial_o[((head0 + g) * p.splits + split) * DH + dim] = sum;
  }
  if (tid < G) {
    float* ml = p.partial_ml + ((head0 + tid) * p.splits + split) * 2;
    ml[0] = m[tid];
    ml[1] = l[tid];
  }

  // the last block of this (token, kv head) to get here merges the splits
  __threadfence();
  __syncthreads();
  if (tid == 0) {
    int* counter = p.counters + token * p.Hkv + kvh;
    const int arrived = atomicAdd(counter, 1);
    *flag = (arrived == used - 1) ? 1 : 0;
    if (arrived == used - 1) *counter = 0;          // left at zero for the next step
  }
  __syncthreads();
  if (*flag == 0) return;
  __threadfence();
  for (int index = tid; index < G * DH; index += MX_THREADS) {
    const int g = index / DH;
    const int dim = index - g * DH;
    const float* ml = p.partial_ml + (head0 + g) * p.splits * 2;
    const float* o = p.partial_o + (head0 + g) * (long)p.splits * DH;
    float maximum = -INFINITY;
    for (int s = 0; s < used; ++s) maximum = fmaxf(maximum, ml[2 * s]);
    float denominator = 0.f, sum = 0.f;
    for (int s = 0; s < used; ++s) {
      const float weight = __expf(ml[2 * s] - maximum);
      denominator += weight * ml[2 * s + 1];
      sum += weight * o[(long)s * DH + dim];
    }
    p.attn_out[token * p.out_ld + (long)(kvh * G + g) * DH + dim] = (bf16_t)(sum / denominator);
  }
}

// One step of the selective scan for (token, head, tile of state rows); see ssm_scan_kernel.
__device__ void mixer_ssm_block(const MixerParams& p, int block) {
  const int tile = block % p.p_tiles;
  const int head = (block / p.p_tiles) % p.H;
  const long token = block / (p.p_tiles * p.H);
  const int R = p.R;
  const int rows_per_block = MX_THREADS / R;
  const int row_in_block = threadIdx.x / R;
  const int r = threadIdx.x - row_in_block * R;
  const int pi = tile * rows_per_block + row_in_block;
  const bool active = pi < p.P;
  const int group = head / (p.H / p.G);
  const int N = p.N;
  const bf16_t* row = p.u + token * p.u_ld;
  float* s_row = p.ssm_state + (((long)p.slot_ids[token] * p.H + head) * p.P + (active ? pi : 0)) * N;
  const float delta = softplus_f((float)row[p.dt_col + head] + p.dt_bias[head]);
  const float decay = expf(delta * p.A[head]);
  const float x = active ? (float)row[p.x_col + head * p.P + pi] : 0.f;
  const bf16_t* b_row = row + p.x_col + p.H * p.P + group * N;
  const bf16_t* c_row = b_row + p.G * N;
  const float dx = delta * x;
  float partial = 0.f;
#pragma unroll
  for (int i = 0; i < MX_SCAN_PER_THREAD; ++i) {
    const int n = r + i * R;
    if (active && n < N) {
      const float next = decay * s_row[n] + dx * (float)b_row[n];
      s_row[n] = next;
      partial += next * (float)c_row[n];
    }
  }
  for (int offset = R / 2; offset > 0; offset >>= 1) partial += __shfl_xor(partial, offset, WAVE);
  if (active && r == 0) {
    const float y = partial + p.D[head] * x;
    const long column = (long)head * p.P + pi;
    if (p.ssm_y) p.ssm_y[token * (long)(p.H * p.P) + column] = y;
    else p.ssm_out[token * p.out_ld + column] = (bf16_t)(y * silu_f((float)row[p.z_col + column]));
  }
}

template <int DH, int G>
__global__ void __launch_bounds__(MX_THREADS) mixer_decode_kernel(MixerParams p) {
  __shared__ float s_lds[G][MX_MAX_SPLIT];
  __shared__ float red[MX_WAVES][8];
  __shared__ float acc_lds[MX_WAVES * G * DH];
  __shared__ int flag;
  if ((int)blockIdx.x < p.attention_blocks)
    mixer_attention_block<DH, G>(p, blockIdx.x, s_lds, red, acc_lds, &flag);
  else
    mixer_ssm_block(p, blockIdx.x - p.attention_blocks);
}

extern "C" int mi_mixer_decode(const void* u, long u_ld, int M, int Hq, int Hkv, int dh, int q_col, int k_col,
                               int v_col, const float* inv_freq, int rotary_dim, void* k_base, void* v_base,
                               long page_stride, int page_size, const int* block_tables, int max_pages,
                               const int* positions, const int* slot_mapping, float scale, int window,
                               int split_keys, int splits, float* partial_o, float* partial_ml, int* counters,
                               int H, int P, int N, int G, int z_col, int x_col, int dt_col, const float* dt_bias,
                               const float* A, const float* D, float* ssm_state, const int* slot_ids,
                               void* attn_out, void* ssm_out, float* ssm_y, long out_ld, hipStream_t stream) {
  if (M <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G != 0)
    return ERR_BAD_ARGUMENT;
  const int group = Hq / Hkv;
  if ((dh != 64 && dh != 128) || group > 8 || page_size % 8 != 0 || split_keys % page_size != 0 ||
      split_keys <= 0 || split_keys > MX_MAX_SPLIT || splits <= 0 || N > WAVE * MX_SCAN_PER_THREAD ||
      u_ld % 8 != 0 || q_col % 8 != 0 || rotary_dim > dh || (rotary_dim & 1))
    return ERR_UNSUPPORTED_SIZE;
  MixerParams p;
  p.u = (const bf16_t*)u;
  p.u_ld = u_ld;
  p.M = M;
  p.Hq = Hq;
  p.Hkv = Hkv;
  p.q_col = q_col;
  p.k_col = k_col;
  p.v_col = v_col;
  p.inv_freq = inv_freq;
  p.rotary_dim = inv_freq ? rotary_dim : 0;
  p.k_base = (bf16_t*)k_base;
  p.v_base = (bf16_t*)v_base;
  p.page_stride = page_stride;
  p.page_size = page_size;
  p.block_tables = block_tables;
  p.max_pages = max_pages;
  p.positions = positions;
  p.slot_mapping = slot_mapping;
  p.scale = scale;
  p.window = window;
  p.split_keys = split_keys;
  p.splits = splits;
  p.partial_o = partial_o;
  p.partial_ml = partial_ml;
  p.counters = counters;
  p.H = H;
  p.P = P;
  p.N = N;
  p.G = G;
  int R = 1;
  while (R < N && R < WAVE) R <<= 1;
  p.R = R;
  const int rows_per_block = MX_THREADS / R;
  p.p_tiles = (P + rows_per_block - 1) / rows_per_block;
  p.z_col = z_col;
  p.x_col = x_col;
  p.dt_col = dt_col;
  p.dt_bias = dt_bias;
  p.A = A;
  p.D = D;
  p.ssm_state = ssm_state;
  p.slot_ids = slot_ids;
  p.attn_out = (bf16_t*)attn_out;
  p.ssm_out = (bf16_t*)ssm_out;
  p.ssm_y = ssm_y;
  p.out_ld = out_ld;
  p.attention_blocks = splits * Hkv * M;
  const long total = (long)p.attention_blocks + (long)p.p_tiles * H * M;
  if (total > 0x7fffffffL) return ERR_UNSUPPORTED_SIZE;
#define MX_CASE(DH_, G_) \
  if (dh == DH_ && group == G_) mixer_decode_kernel<DH_, G_><<<(unsigned)total, MX_THREADS, 0, stream>>>(p);
  MX_CASE(64, 1) MX_CASE(64, 2) MX_CASE(64, 3) MX_CASE(64, 4) MX_CASE(64, 5) MX_CASE(64, 6) MX_CASE(64, 7)
  MX_CASE(64, 8) MX_CASE(128, 1) MX_CASE(128, 2) MX_CASE(128, 3) MX_CASE(128, 4) MX_CASE(128, 5)
  MX_CASE(128, 6) MX_CASE(128, 7) MX_CASE(128, 8)
#undef MX_CASE
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
