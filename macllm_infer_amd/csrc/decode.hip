// Fused kernels for decode steps in bfloat16: every lane of the batch holds one token, the
// batch is small (M <= 64 rows), and a step is bound by weight reads and by the latency of
// each dependent kernel.  Three kernels cover a layer's hot path:
//
//   fused_gemm : out[M, N] = epilogue( prologue(x)[M, K] . W[N, K]^T + bias )
//       prologue  NORM : x = (h + delta0 + delta1) / sqrt(mean(.^2) + eps) * w   (residual add
//                        and RMSNorm; block 0 also writes the summed residual to h_out)
//                 PLAIN: x given in bfloat16
//                 MERGE: x given in bfloat16, but for its first columns, the attended heads, which are
//                        merged here from the partial results that mixer_decode's runs of keys left
//                        (what mixer_merge_kernel does in a launch of its own, sum for sum)
//                 A row scale may follow any prologue that gives x as it is (PLAIN, MERGE): x is then a row of the
//                 residual stream times a norm's weight, rounded to bfloat16 but not yet divided by its root mean
//                 square, and the sums of a row are multiplied by 1 / sqrt(sum of squares / width + eps), from the
//                 partial sums of squares that the RESIDUAL epilogue of the product before left (the norm without
//                 a pass of its own: its statistics in float32, its division applied to float32 sums)
//       epilogue  PLAIN : bfloat16 or float32 (x scale) store
//                 RESIDUAL: the result is added to the float32 residual stream in place, h += result; the new rows
//                        times the next norm's weight go out in bfloat16, and the sums of their squares over the
//                        workgroup's 16 features go to ssq[workgroup][row]
//                 SWIGLU: rows come in tiles of 8 gate rows + 8 up rows; stores SiLU(g)*u
//                 CONV  : rows in [conv_lo, conv_hi) are channels of a causal depthwise conv
//                         with K taps: the new sample joins the request's tail, the tail is
//                         rolled, SiLU(conv) is stored; other rows are stored as they are
//     Each block owns 16 output rows (or 2 or 4 tiles of 16 behind the plain prologue, for steps of
//     many rows: the rows of x then cross the caches once per block and not once per 16 features); its
//     waves split K and feed the matrix cores (v_mfma_f32_16x16x32_bf16: A = 16 weight rows x 32 k,
//     B = 16 batch rows x 32 k, both contiguous in k), then sum their partial tiles through LDS.
//
//   shared_rows_gemm : the same product behind the plain prologue where the rows of x, fetched by every wave
//     of fused_gemm, cross the caches as often as the weights (16 rows) or several times as often: a workgroup's
//     four waves own tiles of 16 features each and walk the same columns, which go through LDS once a
//     workgroup.  Epilogues: float32 slabs over K (to 128 rows), SWIGLU, CONV or plain bfloat16 rows.
//
//   mixer_decode : one launch with two kinds of blocks
//       attention blocks: one per (token, kv head): rotation of q and of the new key, the write
//         of the new K and V into their cache cell, and attention over the request's pages with
//         an online softmax per wave, merged through LDS;
//       state-space blocks: one step of the selective scan from and into the slot state, D skip
//         and the SiLU(z) gate.
//
// Formulas and their reference lines are the ones cited in common.hip, attention.hip and
// mamba2.hip; these kernels only change what runs together.
#include "common.h"
#include "attn_mfma.h"

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

#define FG_PAD 8

enum { PRO_NORM = 0, PRO_PLAIN = 1, PRO_MERGE = 2 };
#define MERGE_AT_ONCE 8      // runs of keys asked for at once by a merge (mixer_merge_kernel and the MERGE prologue)
enum { EPI_PLAIN = 0, EPI_SWIGLU = 1, EPI_CONV = 2, EPI_RESIDUAL = 3 };
#define SSQ_PARTS 16         // threads that share the sum of a row's partial sums of squares
#define SSQ_EARLY 12         // partial sums a thread asks for before the products (rows of up to 3,072 at 16 rows)

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
  int w_tiled;
  // MERGE prologue: partial [M, heads, runs, head_dim + 2] = (maximum, normalizer, sums) per run of keys
  const float* partial;
  const int* positions;
  int merge_heads, merge_dh, merge_runs, merge_run_keys, merge_page, merge_window;
  // RESIDUAL epilogue: h [M, N] float32 (in place), hb [M, hb_ld] bfloat16 = h * next_w[n], ssq_out [workgroups, 16 MT]
  float* res_h;
  bf16_t* res_hb;
  long res_hb_ld;
  const float* res_w;
  float* ssq_out;
  // row scale: ssq_in [ssq_blocks, 16 MT] partial sums of squares of rows of ssq_width elements
  const float* ssq_in;
  int ssq_blocks, ssq_width;
  float ssq_eps;
  // both tables of partial sums of squares have rows of ssq_ld floats: one per row of the step, to a multiple of 16
  int ssq_ld;
  // the step's rows dealt out to row_tiles workgroups per tile of features (1: every workgroup takes them all)
  int row_tiles;
};

// What is left of a step for a workgroup that takes `rows` of its rows from row0 on (plain prologue).
__device__ __forceinline__ void take_rows(FusedGemmParams& p, int row0, int rows) {
  if (p.x) p.x += (long)row0 * p.x_ld;
  if (p.out) p.out = p.out_f32 ? (void*)(reinterpret_cast<float*>(p.out) + (long)row0 * p.out_ld)
                               : (void*)(reinterpret_cast<bf16_t*>(p.out) + (long)row0 * p.out_ld);
  if (p.slot_ids) p.slot_ids += row0;
  if (p.res_h) {
    p.res_h += (long)row0 * p.N;
    p.res_hb += (long)row0 * p.res_hb_ld;
    p.ssq_out += row0;
  }
  if (p.ssq_in) p.ssq_in += row0;
  p.M = min(rows, p.M - row0);
}

__device__ __forceinline__ float round_bf16(float v) { return (float)(bf16_t)v; }

template <int MT, int PRO, int EPI, int FG_WAVES, int NT, bool ROW_TILES = false>
__global__ void __launch_bounds__(FG_WAVES * WAVE) fused_gemm_kernel(FusedGemmParams whole_step) {
  static_assert(NT == 1 || PRO == PRO_PLAIN, "several feature tiles a workgroup: plain prologue only");
  // Row tiles: a workgroup takes MT tiles of 16 rows of the step and row_tiles workgroups share a tile of
  // features.  Workgroups go to the eight dies in turn and each die has a cache of its own, so those that share
  // weights are given numbers that are 8 apart and follow each other: the weights leave memory once.
  FusedGemmParams p = whole_step;
  const int slab_rows = p.M;
  int block_x = blockIdx.x;
  int ssq_rows = p.ssq_ld;              // rows of the tables of partial sums of squares from this workgroup's first row on
  if (ROW_TILES) {
    static_assert(!ROW_TILES || (PRO == PRO_PLAIN && NT == 1), "rows dealt out: plain prologue, one tile of features");
    const int die = block_x % 8, turn = block_x / 8;
    block_x = (turn / p.row_tiles) * 8 + die;
    if (block_x * 16 * NT >= p.N) return;
    const int row0 = (turn % p.row_tiles) * MT * 16;
    ssq_rows -= row0;
    take_rows(p, row0, MT * 16);
  }
  static_assert(PRO != PRO_MERGE || EPI == EPI_PLAIN || EPI == EPI_RESIDUAL, "the merge prologue comes with the plain or the residual epilogue");
  static_assert(EPI != EPI_RESIDUAL || (NT == 1 && PRO != PRO_NORM), "the residual epilogue: one tile of features, rows given as they are");
  constexpr int FG_THREADS = FG_WAVES * WAVE;
  extern __shared__ __align__(16) unsigned char smem[];
  const int K = p.K;
  const int staged = PRO == PRO_NORM ? K : PRO == PRO_MERGE ? p.merge_heads * p.merge_dh : 0;   // columns of x kept in LDS
  const int staged_rows = min(p.M, MT * 16);          // and its rows: the step's own (a tile's rows past M read row M - 1)
  const int ldx = staged + FG_PAD;
  bf16_t* xs = reinterpret_cast<bf16_t*>(smem);
  float* red = reinterpret_cast<float*>(smem + (staged ? (size_t)staged_rows * ldx * sizeof(bf16_t) : 0));
  float* tile = red + FG_WAVES * MT * 256;
  float* ssq_parts = tile + 16 * MT * 16;            // [SSQ_PARTS][16 MT]
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;

  const int n0 = block_x * 16 * NT;
  const int q = lane / 16;
  const int r = lane % 16;
  // W is row-major [N, K], or (w_tiled) in the order of the matrix-core fragments: [N / 16, K / 32, 64 lanes, 8],
  // lane (q, r) of tile (n, c) holding W[16 n + r, 32 c + 8 q ..]: a wave's load then is one run of 1 KiB
  const bf16_t* w_row[NT];
  const long w_step = p.w_tiled ? 512 : 32;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
    w_row[nt] = p.w_tiled ? p.W + (long)min(block_x * NT + nt, (p.N + 15) / 16 - 1) * (K / 32) * 512 + lane * 8
                          : p.W + (long)min(n0 + 16 * nt + r, p.N - 1) * K + 8 * q;
  // wave w takes a contiguous run of k-chunks (of 32), so that its loads cover whole cache lines
  // (a grid with several rows splits K among them: row y takes a run of chunks and writes its partial
  // sums, float32, into slab y of the output; whoever reads them adds the slabs up)
  const int chunks = K / 32;
  const int per_split = (chunks + (int)gridDim.y - 1) / (int)gridDim.y;
  const int split_first = (int)blockIdx.y * per_split;
  const int split_end = min(split_first + per_split, chunks);
  const int per_wave = (max(split_end - split_first, 0) + FG_WAVES - 1) / FG_WAVES;
  const int first_chunk = split_first + wave * per_wave;
  const int iterations = max(0, min(per_wave, split_end - first_chunk));
  // fragments of a wave in flight at once: few of them with 8 waves (long K, many workgroups a CU:
  // the registers saved buy more waves, which hide more than deeper batches do)
  constexpr int BATCH = (FG_WAVES == 8 || NT > 1) ? 4 : 8;
  bf16x8_t a[BATCH][NT];

  // The outputs this thread finishes in the epilogue: element tid + j * FG_THREADS of the block's
  // MT x (16 rows x 16 features), all of one feature.  The slots of their rows are asked for before
  // everything else, because the addresses of their conv tails wait for them.
  constexpr int EPT = (MT * 256 + FG_THREADS - 1) / FG_THREADS;        // outputs a thread finishes
  constexpr int TAILS = (MT == 1 && FG_THREADS == 256) ? 8 : 3;         // tail samples kept per output
  const int tail_n = n0 + 4 * ((tid % 64) / 16) + (tid % 256) / 64;      // in the first tile; 16 more per tile
  int tail_slot[EPT] = {};
  bool tail_wanted[NT] = {};
  if (EPI == EPI_CONV && p.conv_k >= 2 && p.conv_k <= TAILS + 1) {
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) tail_wanted[nt] = tail_n + 16 * nt >= p.conv_lo && tail_n + 16 * nt < p.conv_hi;
#pragma unroll
    for (int j = 0; j < EPT; ++j)
      tail_slot[j] = p.slot_ids[min(((tid + j * FG_THREADS) / 256) * 16 + tid % 16, p.M - 1)];
  }

  // the elements of the residual stream that this thread will add to (RESIDUAL) are asked for up here as well
  constexpr int PARTS = SSQ_PARTS / MT;               // PARTS * 16 MT threads: within the 256 of four waves

  float res_old[EPT] = {};
  float res_weight = 0.f;
  if (EPI == EPI_RESIDUAL) {
    const int n_mine = min(n0 + 4 * ((tid % 64) / 16) + (tid % 256) / 64, p.N - 1);
    res_weight = p.res_w[n_mine];
#pragma unroll
    for (int j = 0; j < EPT; ++j)
      res_old[j] = p.res_h[(long)min(((tid + j * FG_THREADS) / 256) * 16 + tid % 16, p.M - 1) * p.N + n_mine];
  }

  // Loads come back in the order they were asked for, and a wait counts all of them.  The rows
  // to normalize (written by the kernels before, so close by) are asked for first, two rows a
  // wave and without a branch between the loads (a row past M or an absent delta reads a valid
  // address and is not used); the weights, which stream from memory, right after: the norm is
  // computed while the weights are on their way.
  constexpr int MAXV = FG_WAVES == 8 ? 8 : 4;       // 8 waves are launched for K > 1024 only
  const bool in_registers = PRO == PRO_NORM && K <= MAXV * WAVE * 4;
  floatx4 hv[2][MAXV];
  bf16x4_t d0v[2][MAXV], d1v[2][MAXV];
  floatx4 norm_weight[MAXV];
  const bool has0 = p.delta0 != nullptr, has1 = p.delta1 != nullptr;
  auto load_pair = [&](int m0, int pair) {
    long at[2][MAXV];
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int i = 0; i < MAXV; ++i)
        at[tt][i] = (long)min(m0 + wave + (2 * pair + tt) * FG_WAVES, p.M - 1) * K + min(lane * 4 + i * WAVE * 4, K - 4);
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int i = 0; i < MAXV; ++i) hv[tt][i] = *reinterpret_cast<const floatx4*>(p.h_in + at[tt][i]);
    if (has0) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < MAXV; ++i) d0v[tt][i] = *reinterpret_cast<const bf16x4_t*>(p.delta0 + at[tt][i]);
    }
    if (has1) {
#pragma unroll
      for (int tt = 0; tt < 2; ++tt)
#pragma unroll
        for (int i = 0; i < MAXV; ++i) d1v[tt][i] = *reinterpret_cast<const bf16x4_t*>(p.delta1 + at[tt][i]);
    }
  };
  // MERGE: an item is 8 dims of one head of one token; its runs' (maximum, normalizer, 8 sums) are asked for
  // before the weights, MERGE_AT_ONCE runs at once and before it is known how many of them hold keys (the
  // position is on its way too; what a run without keys left in its place is read and not used)
  const int merge_items = PRO == PRO_MERGE ? p.M * (staged / 8) : 0;
  float run_max[MERGE_AT_ONCE], run_norm[MERGE_AT_ONCE];
  float2 run_sums[MERGE_AT_ONCE][4];
  int merge_position = 0;
  auto merge_ask = [&](int item, int first_run) {
    item = min(item, merge_items - 1);
    const int token = item / (staged / 8);
    const int column = (item - token * (staged / 8)) * 8;             // head * dh + dim
    const int head = column / p.merge_dh;
    const float* runs = p.partial + ((long)token * p.merge_heads + head) * p.merge_runs * (long)(p.merge_dh + 2);
    if (first_run == 0) merge_position = p.positions[token];
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j) {
      const float* run = runs + (long)min(first_run + j, p.merge_runs - 1) * (p.merge_dh + 2);
      run_max[j] = run[0];
      run_norm[j] = run[1];
#pragma unroll
      for (int i = 0; i < 4; ++i) run_sums[j][i] = *reinterpret_cast<const float2*>(run + 2 + (column - head * p.merge_dh) + 2 * i);
    }
  };
  if (PRO == PRO_MERGE) merge_ask(tid, 0);
  if (in_registers) {
    load_pair(0, 0);
#pragma unroll
    for (int i = 0; i < MAXV; ++i)
      norm_weight[i] = *reinterpret_cast<const floatx4*>(p.norm_w + min(lane * 4 + i * WAVE * 4, K - 4));
  }
#pragma unroll
  for (int j = 0; j < BATCH; ++j)      // no condition around these loads: a wave without chunks reads the last one
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
      a[j][nt] = *reinterpret_cast<const bf16x8_t*>(w_row[nt] + min(first_chunk + min(j, max(iterations, 1) - 1), chunks - 1) * w_step);
  // the partial sums of squares of the rows (row scale), 16 MT rows by SSQ_PARTS threads each: asked for behind the
  // weights and behind the step's rows of the first round of products (ahead of them, these dozen loads of what the
  // kernel before has just written on other dies hold back what the products wait for: a decode step of 8 rows took
  // 1.383 ms with the sums first, 1.364 with them behind the weights, 1.355 behind the rows too) and not added up
  // before the products are done; past the last workgroup's sums, a valid address
  float ssq_early[SSQ_EARLY] = {};
  auto ask_ssq = [&]() {
    const int last = p.ssq_blocks - 1;
    const int row = min(tid % (16 * MT), ssq_rows - 1);
#pragma unroll
    for (int i = 0; i < SSQ_EARLY; ++i)
      ssq_early[i] = p.ssq_in[(long)min(tid / (16 * MT) + i * PARTS, last) * p.ssq_ld + row];
  };
  if (PRO == PRO_PLAIN && p.ssq_in && iterations == 0) ask_ssq();          // a wave without a run of K has no round
  if (PRO == PRO_NORM) {
    // one wave per row, two rows at a time: the rows are read once into registers (K <= 2048),
    // their sums of squares reduced in float32, and the normalized rows written in bfloat16
    for (int m0 = 0; m0 < MT * 16; m0 += FG_WAVES * 4) {
#pragma unroll
      for (int pair = 0; pair < 2; ++pair) {
        if (in_registers && (m0 > 0 || pair > 0) && m0 + wave + 2 * pair * FG_WAVES < p.M) load_pair(m0, pair);
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
          const int m = m0 + wave + (2 * pair + tt) * FG_WAVES;
          if (m >= staged_rows) continue;
          bf16_t* x_row = xs + (long)m * ldx;
          const float* h_row = p.h_in + (long)m * K;
          auto row_value = [&](int k) {
            floatx4 value = *reinterpret_cast<const floatx4*>(h_row + k);
            if (has0) {
              const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(p.delta0 + (long)m * K + k);
#pragma unroll
              for (int j = 0; j < 4; ++j) value[j] += (float)d[j];
            }
            if (has1) {
              const bf16x4_t d = *reinterpret_cast<const bf16x4_t*>(p.delta1 + (long)m * K + k);
#pragma unroll
              for (int j = 0; j < 4; ++j) value[j] += (float)d[j];
            }
            return value;
          };
          float sum_squares = 0.f;
          if (in_registers) {
#pragma unroll
            for (int i = 0; i < MAXV; ++i) {
#pragma unroll
              for (int j = 0; j < 4; ++j) {
                float value = hv[tt][i][j];
                if (has0) value += (float)d0v[tt][i][j];
                if (has1) value += (float)d1v[tt][i][j];
                hv[tt][i][j] = value;
                if (lane * 4 + i * WAVE * 4 < K) sum_squares += value * value;
              }
            }
          } else {
            for (int k = lane * 4; k < K; k += WAVE * 4) {
              const floatx4 value = row_value(k);
#pragma unroll
              for (int j = 0; j < 4; ++j) sum_squares += value[j] * value[j];
            }
          }
          sum_squares = wave_sum(sum_squares);
          const float inverse = 1.0f / sqrtf(sum_squares / (float)K + p.eps);
          auto finish = [&](int k, const floatx4& value, const floatx4& w) {
            if (block_x == 0 && p.h_out) *reinterpret_cast<floatx4*>(p.h_out + (long)m * K + k) = value;
            bf16x4_t packed;
#pragma unroll
            for (int j = 0; j < 4; ++j) packed[j] = (bf16_t)(value[j] * inverse * w[j]);
            *reinterpret_cast<bf16x4_t*>(x_row + k) = packed;
          };
          if (in_registers) {
#pragma unroll
            for (int i = 0; i < MAXV; ++i) {
              const int k = lane * 4 + i * WAVE * 4;
              if (k < K) finish(k, hv[tt][i], norm_weight[i]);
            }
          } else {
            for (int k = lane * 4; k < K; k += WAVE * 4)
              finish(k, row_value(k), *reinterpret_cast<const floatx4*>(p.norm_w + k));
          }
        }
      }
    }
    __syncthreads();
  }
  if (PRO == PRO_MERGE) {
    // out[token, head, :] = sum_s exp(m_s - m) o_s / sum_s exp(m_s - m) l_s over the runs that hold keys,
    // in the order and with the roundings of mixer_merge_kernel
    for (int item = tid; item < merge_items; item += FG_THREADS) {
      if (item != tid) merge_ask(item, 0);
      int first_key = 0;
      if (p.merge_window > 0 && merge_position - p.merge_window + 1 > 0) first_key = merge_position - p.merge_window + 1;
      const int base_key = (first_key / p.merge_page) * p.merge_page;
      const int used = min(p.merge_runs, (merge_position - base_key) / p.merge_run_keys + 1);
      float maximum = -INFINITY, denominator = 0.f, sums[8] = {};
      for (int s0 = 0; s0 < used; s0 += MERGE_AT_ONCE) {
        if (s0 > 0) merge_ask(item, s0);
#pragma unroll
        for (int j = 0; j < MERGE_AT_ONCE; ++j) {
          if (s0 + j < used) {
            const float larger = fmaxf(maximum, run_max[j]);
            const float keep = __builtin_amdgcn_exp2f(maximum - larger);          // 0 the first time; units of log2
            const float weight = __builtin_amdgcn_exp2f(run_max[j] - larger);
            denominator = denominator * keep + weight * run_norm[j];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              sums[2 * i] = sums[2 * i] * keep + weight * run_sums[j][i].x;
              sums[2 * i + 1] = sums[2 * i + 1] * keep + weight * run_sums[j][i].y;
            }
            maximum = larger;
          }
        }
      }
      const int token = item / (staged / 8);
      const int column = (item - token * (staged / 8)) * 8;
      bf16x8_t packed;
#pragma unroll
      for (int i = 0; i < 8; ++i) packed[i] = (bf16_t)(sums[i] / denominator);
      *reinterpret_cast<bf16x8_t*>(xs + (long)token * ldx + column) = packed;
    }
    __syncthreads();
  }

  // the conv tails of those outputs are asked for now, behind the weights; no branch between the
  // loads either (a row past M reads the last row's tail and is not used)
  bf16_t tail_values[NT][EPT][TAILS];
  float tap_values[NT][TAILS + 1];
  float tap_bias[NT] = {};
  bool tail_ready[NT] = {};
  if (EPI == EPI_CONV) {
#pragma unroll
    for (int j = 0; j < EPT; ++j) asm volatile("" : "+v"(tail_slot[j]));   // keeps every use of the slots (and their wait) down here
  }
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (!tail_wanted[nt]) continue;
    const int channels = p.conv_hi - p.conv_lo;
    const int channel = tail_n + 16 * nt - p.conv_lo;
#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const bf16_t* tail = p.conv_state + (long)tail_slot[j] * (p.conv_k - 1) * channels + channel;
#pragma unroll
      for (int k = 0; k < TAILS; ++k) tail_values[nt][j][k] = tail[(long)min(k, p.conv_k - 2) * channels];
    }
#pragma unroll
    for (int k = 0; k < TAILS + 1; ++k) tap_values[nt][k] = p.conv_w[(long)channel * p.conv_k + min(k, p.conv_k - 1)];
    if (p.conv_b) tap_bias[nt] = p.conv_b[channel];
    tail_ready[nt] = true;
  }

  // the product: eight weight fragments are requested before the first is used, so that a
  // wave keeps eight 1 KiB loads in flight
  floatx4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  for (int first = 0; first < iterations; first += BATCH) {
    if (first > 0) {
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        const int c = first_chunk + min(first + j, iterations - 1);
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) a[j][nt] = *reinterpret_cast<const bf16x8_t*>(w_row[nt] + c * w_step);
      }
    }
    bf16x8_t b[BATCH][MT];
    if (PRO == PRO_PLAIN || PRO == PRO_MERGE) {
#pragma unroll
      for (int j = 0; j < BATCH; ++j) {
        const int c = first_chunk + min(first + j, iterations - 1);
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          const int m = min(mt * 16 + r, p.M - 1);
          if (PRO == PRO_MERGE && c * 32 < staged) b[j][mt] = *reinterpret_cast<const bf16x8_t*>(xs + (long)m * ldx + c * 32 + 8 * q);
          else b[j][mt] = *reinterpret_cast<const bf16x8_t*>(p.x + (long)m * p.x_ld + c * 32 + 8 * q);
        }
      }
    }
    if (PRO == PRO_PLAIN && first == 0 && p.ssq_in) ask_ssq();         // (a row scale comes with the plain prologue only)
    // no branch around a product: under a condition the compiler moves the fragment's load into the
    // branch and waits for it there, one at a time; a fragment past the end is read again (clamped
    // above) and multiplied as zeros
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int c = first_chunk + min(first + j, iterations - 1);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const floatx4 weights = first + j < iterations ? *reinterpret_cast<const floatx4*>(&a[j][nt]) : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          bf16x8_t operand;
          if (PRO == PRO_NORM) operand = *reinterpret_cast<const bf16x8_t*>(xs + (long)min(mt * 16 + r, p.M - 1) * ldx + c * 32 + 8 * q);
          else operand = b[j][mt];
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8_t*>(&weights), operand, acc[nt][mt], 0, 0, 0);
        }
      }
    }
  }
  if (p.ssq_in && tid < PARTS * 16 * MT) {          // read behind the barrier below
    const int part = tid / (16 * MT);
    float sum = 0.f;
#pragma unroll
    for (int i = 0; i < SSQ_EARLY; ++i) sum += part + i * PARTS < p.ssq_blocks ? ssq_early[i] : 0.f;
    // rows wider than SSQ_EARLY sums a thread: the rest now
    for (int b = part + SSQ_EARLY * PARTS; b < p.ssq_blocks; b += PARTS) sum += p.ssq_in[(long)b * p.ssq_ld + min(tid % (16 * MT), ssq_rows - 1)];
    ssq_parts[tid] = sum;
  }
  // the waves' partial tiles are summed through LDS and finished, one tile of 16 features after the other
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int tile_n0 = n0 + 16 * nt;
    if (nt > 0) __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[(wave * MT + mt) * 256 + i * 64 + lane] = acc[nt][mt][i];
    __syncthreads();

#pragma unroll
    for (int j = 0; j < EPT; ++j) {
      const int index = tid + j * FG_THREADS;
      if (index >= MT * 256) continue;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < FG_WAVES; ++w) v += red[w * MT * 256 + index];
      const int mt = index / 256;
      const int i = (index % 256) / 64;
      const int l = index % 64;
      const int n_local = 4 * (l / 16) + i;
      const int n = tile_n0 + n_local;
      const int m = mt * 16 + (l % 16);
      if (p.ssq_in) {                          // the norm's division, on the float32 sums
        float squares = 0.f;
#pragma unroll
        for (int part = 0; part < PARTS; ++part) squares += ssq_parts[part * (16 * MT) + m];
        v *= 1.0f / sqrtf(squares / (float)p.ssq_width + p.ssq_eps);
      }
      if (p.bias && n < p.N && blockIdx.y == 0) v += p.bias[n];
      if (EPI == EPI_SWIGLU) {
        tile[n_local * (MT * 16) + m] = v;
        continue;
      }
      if (EPI == EPI_RESIDUAL) {
        float square = 0.f;
        if (n < p.N && m < p.M) {
          const float updated = res_old[j] + v * p.out_scale;
          p.res_h[(long)m * p.N + n] = updated;
          p.res_hb[(long)m * p.res_hb_ld + n] = (bf16_t)(updated * res_weight);
          square = updated * updated;
        }
        tile[n_local * (MT * 16) + m] = square;
        continue;
      }
      if (n >= p.N || m >= p.M) continue;
      if (EPI == EPI_CONV && n >= p.conv_lo && n < p.conv_hi) {
        const int channel = n - p.conv_lo;
        const int channels = p.conv_hi - p.conv_lo;
        const int taps = p.conv_k;
        bf16_t* tail = p.conv_state + (long)(tail_ready[nt] ? tail_slot[j] : p.slot_ids[m]) * (taps - 1) * channels + channel;
        const bf16_t sample = (bf16_t)v;
        float sum;
        if (tail_ready[nt]) {                   // taps, bias and tail are in registers already
          sum = tap_bias[nt];
#pragma unroll
          for (int k = 0; k < TAILS; ++k) {
            if (k < taps - 1) {
              sum += tap_values[nt][k] * (float)tail_values[nt][j][k];
              if (k > 0) tail[(long)(k - 1) * channels] = tail_values[nt][j][k];   // roll the tail by one
            }
          }
          float last_tap = tap_values[nt][0];
#pragma unroll
          for (int k = 1; k < TAILS + 1; ++k) last_tap = k == taps - 1 ? tap_values[nt][k] : last_tap;
          sum += last_tap * (float)sample;
        } else {
          sum = p.conv_b ? p.conv_b[channel] : 0.f;
          for (int k = 0; k < taps - 1; ++k) {
            const bf16_t old = tail[(long)k * channels];
            sum += p.conv_w[channel * taps + k] * (float)old;
            if (k > 0) tail[(long)(k - 1) * channels] = old;       // roll the tail by one
          }
          sum += p.conv_w[channel * taps + taps - 1] * (float)sample;
        }
        if (taps > 1) tail[(long)(taps - 2) * channels] = sample;
        reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + n] = (bf16_t)silu_f(sum);
      } else if (p.out_f32) {
        reinterpret_cast<float*>(p.out)[((long)blockIdx.y * slab_rows + m) * p.out_ld + n] = v * p.out_scale;
      } else {
        reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + n] = (bf16_t)(v * p.out_scale);
      }
    }
    if (EPI == EPI_RESIDUAL) {
      __syncthreads();
      if (tid < min(MT * 16, ssq_rows)) {
        float squares = 0.f;
#pragma unroll
        for (int f = 0; f < 16; ++f) squares += tile[f * (MT * 16) + tid];
        p.ssq_out[(long)block_x * p.ssq_ld + tid] = squares;
      }
    }
    if (EPI == EPI_SWIGLU) {
      __syncthreads();
      const int half_rows = p.N / 2;
      for (int index = tid; index < 8 * MT * 16; index += FG_THREADS) {
        const int i = index / (MT * 16);
        const int m = index % (MT * 16);
        const int column = (block_x * NT + nt) * 8 + i;
        if (m >= p.M || column >= half_rows) continue;
        const float gate = round_bf16(tile[i * (MT * 16) + m]);
        const float up = round_bf16(tile[(8 + i) * (MT * 16) + m]);
        reinterpret_cast<bf16_t*>(p.out)[(long)m * p.out_ld + column] = (bf16_t)(silu_f(gate) * up);
      }
    }
  }
}

static int fused_gemm_waves(int K) { return K / 32 > 32 ? 8 : 4; }   // 8 waves split a long K

// staged: the columns of x the prologue keeps in LDS (all of K behind the norm, the merged heads behind the
// merge), for the M rows of the step
static size_t fused_gemm_lds(int MT, int pro, int K, int M, int staged = 0) {
  size_t bytes = (size_t)fused_gemm_waves(K) * MT * 256 * sizeof(float) + (size_t)16 * MT * 16 * sizeof(float) +
                 (size_t)SSQ_PARTS * 16 * MT * sizeof(float);
  if (pro == PRO_NORM) staged = K;
  if (pro != PRO_PLAIN) bytes += (size_t)(M < MT * 16 ? M : MT * 16) * (staged + FG_PAD) * sizeof(bf16_t);
  return bytes;
}

// feature_tiles: how many tiles of 16 output features a workgroup owns (1, 2 or 4).  With one, the rows of x
// cross the caches once per 16 features, which is what bounds a step of many rows; with more, fewer
// workgroups (of four waves) each keep more weight fragments in flight.  Plain prologue only.
template <int MT>
static int launch_fused_gemm(const FusedGemmParams& p, int pro, int epi, hipStream_t stream, int k_splits = 1,
                             int feature_tiles = 1) {
  const size_t lds = fused_gemm_lds(MT, pro, p.K, p.M, pro == PRO_MERGE ? p.merge_heads * p.merge_dh : 0);
  if (feature_tiles > 1) {
    if (pro != PRO_PLAIN || (feature_tiles != 2 && feature_tiles != 4)) return ERR_BAD_ARGUMENT;
    const dim3 blocks((p.N + 16 * feature_tiles - 1) / (16 * feature_tiles), k_splits);
#define FG_WIDE(EPI_)                                                                                  \
  do {                                                                                                 \
    if (feature_tiles == 2) fused_gemm_kernel<MT, PRO_PLAIN, EPI_, 4, 2><<<blocks, 4 * WAVE, lds, stream>>>(p); \
    else fused_gemm_kernel<MT, PRO_PLAIN, EPI_, 4, 4><<<blocks, 4 * WAVE, lds, stream>>>(p);           \
  } while (0)
    if (epi == EPI_PLAIN) FG_WIDE(EPI_PLAIN);
    else if (epi == EPI_SWIGLU) FG_WIDE(EPI_SWIGLU);
    else if (epi == EPI_CONV) FG_WIDE(EPI_CONV);
    else return ERR_BAD_ARGUMENT;
#undef FG_WIDE
    return 0;
  }
  const int feature_blocks = (p.N + 15) / 16;
  const dim3 blocks(p.row_tiles > 1 ? (feature_blocks + 7) / 8 * 8 * p.row_tiles : feature_blocks, k_splits);
  const int waves = fused_gemm_waves(p.K / k_splits);
#define FG_LAUNCH(PRO_, EPI_)                                                                      \
  do {                                                                                             \
    if (waves == 8) fused_gemm_kernel<MT, PRO_, EPI_, 8, 1><<<blocks, 8 * WAVE, lds, stream>>>(p); \
    else fused_gemm_kernel<MT, PRO_, EPI_, 4, 1><<<blocks, 4 * WAVE, lds, stream>>>(p);            \
  } while (0)
#define FG_LAUNCH_ROWS(EPI_)                                                                                  \
  do {                                                                                                        \
    if (waves == 8) fused_gemm_kernel<MT, PRO_PLAIN, EPI_, 8, 1, true><<<blocks, 8 * WAVE, lds, stream>>>(p); \
    else fused_gemm_kernel<MT, PRO_PLAIN, EPI_, 4, 1, true><<<blocks, 4 * WAVE, lds, stream>>>(p);            \
  } while (0)
  if (p.row_tiles > 1) {           // MT of 1 or 2: the tiles of a step of up to 64 rows over two workgroups or more
    if (pro != PRO_PLAIN) return ERR_BAD_ARGUMENT;
    if constexpr (MT <= 2) {
      if (epi == EPI_RESIDUAL) FG_LAUNCH_ROWS(EPI_RESIDUAL);
      else if (epi == EPI_PLAIN) FG_LAUNCH_ROWS(EPI_PLAIN);
      else if (epi == EPI_SWIGLU) FG_LAUNCH_ROWS(EPI_SWIGLU);
      else if (epi == EPI_CONV) FG_LAUNCH_ROWS(EPI_CONV);
      else return ERR_BAD_ARGUMENT;
      return 0;
    } else {
      return ERR_BAD_ARGUMENT;
    }
  }
  if (pro == PRO_MERGE && epi == EPI_PLAIN) FG_LAUNCH(PRO_MERGE, EPI_PLAIN);
  else if (pro == PRO_MERGE && epi == EPI_RESIDUAL) FG_LAUNCH(PRO_MERGE, EPI_RESIDUAL);
  else if (pro == PRO_PLAIN && epi == EPI_RESIDUAL) FG_LAUNCH(PRO_PLAIN, EPI_RESIDUAL);
  else if (pro == PRO_NORM && epi == EPI_PLAIN) FG_LAUNCH(PRO_NORM, EPI_PLAIN);
  else if (pro == PRO_NORM && epi == EPI_SWIGLU) FG_LAUNCH(PRO_NORM, EPI_SWIGLU);
  else if (pro == PRO_NORM && epi == EPI_CONV) FG_LAUNCH(PRO_NORM, EPI_CONV);
  else if (pro == PRO_PLAIN && epi == EPI_PLAIN) FG_LAUNCH(PRO_PLAIN, EPI_PLAIN);
  else if (pro == PRO_PLAIN && epi == EPI_SWIGLU) FG_LAUNCH(PRO_PLAIN, EPI_SWIGLU);
  else if (pro == PRO_PLAIN && epi == EPI_CONV) FG_LAUNCH(PRO_PLAIN, EPI_CONV);
  else return ERR_BAD_ARGUMENT;
#undef FG_LAUNCH
#undef FG_LAUNCH_ROWS
  return 0;
}

// The same for a step of p.M rows (up to 64).  row_tiles > 1 (plain prologue, one tile of features a workgroup): the
// tiles of 16 rows are dealt out to that many workgroups per tile of features (64 rows over 4: every workgroup
// multiplies 16 rows), which fills the GPU where a projection has few output features without slabs over K, and
// moves a quarter of the rows through each compute unit; the weights cross the caches row_tiles times.
static int launch_fused_gemm_rows(FusedGemmParams& p, int pro, int epi, hipStream_t stream, int k_splits = 1,
                                  int feature_tiles = 1, int row_tiles = 1) {
  const int step_tiles = (p.M + 15) / 16;
  int MT = step_tiles;
  p.ssq_ld = 16 * step_tiles;
  p.row_tiles = 1;
  if (row_tiles > 1) {
    if (pro != PRO_PLAIN || feature_tiles != 1) return ERR_BAD_ARGUMENT;
    MT = (step_tiles + row_tiles - 1) / row_tiles;
    p.row_tiles = (step_tiles + MT - 1) / MT;
  }
  if (MT == 1) return launch_fused_gemm<1>(p, pro, epi, stream, k_splits, feature_tiles);
  if (MT == 2) return launch_fused_gemm<2>(p, pro, epi, stream, k_splits, feature_tiles);
  if (MT == 3) return launch_fused_gemm<3>(p, pro, epi, stream, k_splits, feature_tiles);
  if (MT == 4) return launch_fused_gemm<4>(p, pro, epi, stream, k_splits, feature_tiles);
  return ERR_UNSUPPORTED_SIZE;
}

// The product in float32 slabs over K for steps of many rows, with the rows shared.  In fused_gemm_kernel every
// wave walks columns of its own, so every wave fetches its own part of the step's rows: at 48 to 64 rows four
// times the bytes of the weights cross the caches (a 5,120 x 21,504 weight at 64 rows: 93 us where the weights
// alone stream in 49).  Here the four waves of a workgroup own NT tiles of 16 features each and walk the same
// columns: the rows of a stage (SR_CHUNKS * 32 columns) are fetched once a workgroup, laid in LDS (two stages,
// one barrier a stage) and read from there by all four, while each wave asks for its next stage's weights before
// it multiplies the current one's.  EPI_PLAIN: float32 slabs over K, one a row of workgroups.  EPI_SWIGLU and
// EPI_CONV: all of K in one workgroup (a gate and up projection or a layer's input projection has features
// enough to fill the GPU); SiLU(gate) * up, or rows in bfloat16 with the conv step of the columns that have
// one (none: plain rows), as in fused_gemm_kernel, with the row scale of a norm left to this product if
// there is one.
constexpr int SR_CHUNKS = 4;
constexpr int SR_LD = SR_CHUNKS * 32 + 8;        // a stage's row in LDS, padded against bank conflicts
// gfx950 gives a workgroup up to 160 KiB of LDS (earlier targets: 64 KiB).  The kernels of this file that size
// their LDS at run time stay within 64 KiB; the two stages of 96 or 128 rows below are static and exceed it,
// which is stated here rather than left to the target.
constexpr int GFX950_LDS_PER_WORKGROUP = 160 * 1024;

template <int MT, int NT, int EPI>
__global__ __launch_bounds__(256) void shared_rows_gemm_kernel(FusedGemmParams p) {
  __shared__ __align__(16) bf16_t stage[2][MT * 16 * SR_LD];
  constexpr int SQUARE_PARTS = MT <= 4 ? 4 : 2;      // threads that add up a row's sums of squares
  __shared__ float squares[SQUARE_PARTS][MT * 16];
  static_assert(sizeof(bf16_t) * 2 * MT * 16 * SR_LD + sizeof(float) * SQUARE_PARTS * MT * 16 <= GFX950_LDS_PER_WORKGROUP,
                "the two stages of the step's rows do not fit a gfx950 workgroup's LDS");
  const int tid = threadIdx.x, wave = tid / WAVE, lane = tid % WAVE, q = lane / 16, r = lane % 16;
  const int tiles = (p.N + 15) / 16;
  const int chunks = p.K / 32;
  const int per_split = (chunks + gridDim.y - 1) / gridDim.y;
  const int first_chunk = blockIdx.y * per_split;
  const int end_chunk = min(first_chunk + per_split, chunks);          // may lie before first_chunk: an empty slab
  const int stages = max(0, end_chunk - first_chunk + SR_CHUNKS - 1) / SR_CHUNKS;
  const int tile0 = (blockIdx.x * 4 + wave) * NT;

  const int w_step = p.w_tiled ? 512 : 32;
  const bf16_t* w_row[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int tile = min(tile0 + nt, tiles - 1);
    w_row[nt] = p.w_tiled ? p.W + (long)tile * chunks * 512 + lane * 8
                          : p.W + (long)min(tile * 16 + r, p.N - 1) * p.K + 8 * q;
  }
  // a thread's pieces of a stage's rows: 8 columns each, 16 pieces a row
  const bf16_t* x_from[MT];
  int x_to[MT];
#pragma unroll
  for (int j = 0; j < MT; ++j) {
    const int piece = tid + j * 256;
    x_from[j] = p.x + (long)min(piece / 16, p.M - 1) * p.x_ld + (piece % 16) * 8;
    x_to[j] = (piece / 16) * SR_LD + (piece % 16) * 8;
  }
  // no condition around a load (a stage or chunk past the end reads the last one again and is multiplied as zeros)
  auto ask_rows = [&](bf16x8_t (&rows)[MT], int s) {
    const int c0 = min(first_chunk + s * SR_CHUNKS, chunks - SR_CHUNKS);
#pragma unroll
    for (int j = 0; j < MT; ++j) rows[j] = *reinterpret_cast<const bf16x8_t*>(x_from[j] + (long)max(c0, 0) * 32);
  };
  auto ask_weights = [&](bf16x8_t (&a)[SR_CHUNKS][NT], int s) {
    const int c0 = max(min(first_chunk + s * SR_CHUNKS, chunks - SR_CHUNKS), 0);
#pragma unroll
    for (int j = 0; j < SR_CHUNKS; ++j)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt)
        a[j][nt] = *reinterpret_cast<const bf16x8_t*>(w_row[nt] + (long)min(c0 + j, chunks - 1) * w_step);
  };
  auto lay_rows = [&](const bf16x8_t (&rows)[MT], int buffer) {
#pragma unroll
    for (int j = 0; j < MT; ++j) *reinterpret_cast<bf16x8_t*>(&stage[buffer][x_to[j]]) = rows[j];
  };

  floatx4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // the stage that starts at chunk c0 (clamped as in the loads) holds the chunks c0 .. c0 + SR_CHUNKS - 1; those
  // outside [from, end_chunk) count as zeros: before `from` where the clamp moved the stage back over chunks
  // that an earlier stage has multiplied already
  auto multiply = [&](const bf16x8_t (&a)[SR_CHUNKS][NT], int s, int buffer) {
    const int wanted = first_chunk + s * SR_CHUNKS;
    const int c0 = max(min(wanted, chunks - SR_CHUNKS), 0);
#pragma unroll
    for (int j = 0; j < SR_CHUNKS; ++j) {
      const bool counts = c0 + j >= wanted && c0 + j < end_chunk;
      bf16x8_t b[MT];
#pragma unroll
      for (int mt = 0; mt < MT; ++mt)
        b[mt] = *reinterpret_cast<const bf16x8_t*>(&stage[buffer][(mt * 16 + r) * SR_LD + j * 32 + 8 * q]);
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        const floatx4 weights = counts ? *reinterpret_cast<const floatx4*>(&a[j][nt]) : floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(*reinterpret_cast<const bf16x8_t*>(&weights), b[mt],
                                                                acc[nt][mt], 0, 0, 0);
      }
    }
  };

  bf16x8_t rows[MT], a_even[SR_CHUNKS][NT], a_odd[SR_CHUNKS][NT];
  ask_rows(rows, 0);
  ask_weights(a_even, 0);
  int slot[MT];                                     // CONV: the rows' conv tails, asked for with the first loads
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) slot[mt] = EPI == EPI_CONV && p.slot_ids ? p.slot_ids[min(mt * 16 + r, p.M - 1)] : 0;
  if (EPI != EPI_PLAIN && p.ssq_in && tid < SQUARE_PARTS * MT * 16) {
    // the rows' sums of squares, which the workgroups of the product before left in parts: a few threads a row
    const int row = tid % (MT * 16);
    float sum = 0.f;
    for (int b = tid / (MT * 16); b < p.ssq_blocks; b += SQUARE_PARTS) sum += p.ssq_in[(long)b * (MT * 16) + row];
    squares[tid / (MT * 16)][row] = sum;
  }
  lay_rows(rows, 0);
  __syncthreads();
  for (int s = 0; s < stages; s += 2) {
    ask_rows(rows, s + 1);
    ask_weights(a_odd, s + 1);
    multiply(a_even, s, 0);
    lay_rows(rows, 1);
    __syncthreads();
    if (s + 1 >= stages) break;
    ask_rows(rows, s + 2);
    ask_weights(a_even, s + 2);
    multiply(a_odd, s + 1, 1);
    lay_rows(rows, 0);
    __syncthreads();
  }

  // lane (q, r) holds features 4 q .. 4 q + 3 of row r of every tile
  float factor[MT];                                 // the norm's division, on the float32 sums
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    factor[mt] = 1.0f;
    if (EPI != EPI_PLAIN && p.ssq_in) {
      const int m = mt * 16 + r;
      float sum = 0.f;
#pragma unroll
      for (int part = 0; part < SQUARE_PARTS; ++part) sum += squares[part][m];
      factor[mt] = 1.0f / sqrtf(sum / (float)p.ssq_width + p.ssq_eps);
    }
  }
  if (EPI == EPI_CONV) {
    // bfloat16 rows; the columns conv_lo .. conv_hi - 1 through the conv step of their channel with the row's
    // tail, which is rolled by one, and SiLU, as in fused_gemm_kernel (no channel is anyone else's)
    bf16_t* out = reinterpret_cast<bf16_t*>(p.out);
    const int channels = p.conv_hi - p.conv_lo;
    const int taps = p.conv_k;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int n = (tile0 + nt) * 16 + 4 * q;
      if (tile0 + nt >= tiles) continue;
      floatx4 bias = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bias[i] = p.bias[min(n + i, p.N - 1)];
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const int m = mt * 16 + r;
        if (m >= p.M) continue;
        const floatx4 v = acc[nt][mt] * factor[mt] + bias;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if (n + i >= p.N) continue;
          if (n + i < p.conv_lo || n + i >= p.conv_hi) {
            out[(long)m * p.out_ld + n + i] = (bf16_t)(v[i] * p.out_scale);
            continue;
          }
          const int channel = n + i - p.conv_lo;
          bf16_t* tail = p.conv_state + (long)slot[mt] * (taps - 1) * channels + channel;
          const bf16_t sample = (bf16_t)v[i];
          float sum = p.conv_b ? p.conv_b[channel] : 0.f;
          for (int k = 0; k < taps - 1; ++k) {
            const bf16_t old = tail[(long)k * channels];
            sum += p.conv_w[channel * taps + k] * (float)old;
            if (k > 0) tail[(long)(k - 1) * channels] = old;       // roll the tail by one
          }
          sum += p.conv_w[channel * taps + taps - 1] * (float)sample;
          if (taps > 1) tail[(long)(taps - 2) * channels] = sample;
          out[(long)m * p.out_ld + n + i] = (bf16_t)silu_f(sum);
        }
      }
    }
    return;
  }
  if (EPI == EPI_SWIGLU) {
    // a tile is 8 gate features, then the 8 up features of the same columns: lanes q = 0, 1 take their up
    // values from the lanes q + 2 and write 4 columns of bfloat16
    bf16_t* out = reinterpret_cast<bf16_t*>(p.out);
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      const int n = (tile0 + nt) * 16 + 4 * q;
      floatx4 bias = {0.f, 0.f, 0.f, 0.f};
      if (p.bias) {
#pragma unroll
        for (int i = 0; i < 4; ++i) bias[i] = p.bias[min(n + i, p.N - 1)];
      }
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const floatx4 v = acc[nt][mt] * factor[mt] + bias;
        floatx4 up;
#pragma unroll
        for (int i = 0; i < 4; ++i) up[i] = __shfl(v[i], (lane + 32) % WAVE);
        const int m = mt * 16 + r;
        const int column = (tile0 + nt) * 8 + 4 * q;
        if (tile0 + nt >= tiles || q >= 2 || m >= p.M) continue;
        bf16x4_t packed;
#pragma unroll
        for (int i = 0; i < 4; ++i) packed[i] = (bf16_t)(silu_f(round_bf16(v[i])) * round_bf16(up[i]));
        bf16_t* to = out + (long)m * p.out_ld + column;
        if (p.out_ld % 4 == 0) {
          *reinterpret_cast<bf16x4_t*>(to) = packed;
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i) to[i] = packed[i];
        }
      }
    }
    return;
  }
  float* slab = reinterpret_cast<float*>(p.out) + (long)blockIdx.y * p.M * p.out_ld;
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    const int n = (tile0 + nt) * 16 + 4 * q;
    if (tile0 + nt >= tiles) continue;
    floatx4 bias = {0.f, 0.f, 0.f, 0.f};
    if (p.bias && blockIdx.y == 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) bias[i] = p.bias[min(n + i, p.N - 1)];
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      const int m = mt * 16 + r;
      if (m >= p.M) continue;
      const floatx4 v = acc[nt][mt] + bias;
      float* to = slab + (long)m * p.out_ld + n;
      if (p.out_ld % 4 == 0 && n + 3 < p.N) {
        *reinterpret_cast<floatx4*>(to) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (n + i < p.N) to[i] = v[i];
      }
    }
  }
}

template <int MT, int EPI>
static int launch_shared_rows(const FusedGemmParams& p, hipStream_t stream, int k_splits, int feature_tiles) {
  const int tiles = (p.N + 15) / 16;
  const dim3 blocks((tiles + 4 * feature_tiles - 1) / (4 * feature_tiles), k_splits);
  if (feature_tiles == 1) shared_rows_gemm_kernel<MT, 1, EPI><<<blocks, 4 * WAVE, 0, stream>>>(p);
  else if (feature_tiles == 2) shared_rows_gemm_kernel<MT, 2, EPI><<<blocks, 4 * WAVE, 0, stream>>>(p);
  else return ERR_BAD_ARGUMENT;
  return 0;
}

// up to 64 rows in tiles of 16; 65 to 128 rows (the slabs only) in 6 or 8 tiles with one tile of features a wave
template <int EPI>
static int launch_shared_rows_for(int M, const FusedGemmParams& p, hipStream_t stream, int k_splits, int feature_tiles) {
  if (M <= 16) return launch_shared_rows<1, EPI>(p, stream, k_splits, feature_tiles);
  if (M <= 32) return launch_shared_rows<2, EPI>(p, stream, k_splits, feature_tiles);
  if (M <= 48) return launch_shared_rows<3, EPI>(p, stream, k_splits, feature_tiles);
  if (M <= 64) return launch_shared_rows<4, EPI>(p, stream, k_splits, feature_tiles);
  if constexpr (EPI == EPI_PLAIN) {
    if (feature_tiles != 1) return ERR_UNSUPPORTED_SIZE;
    const int tiles = (p.N + 15) / 16;
    const dim3 blocks((tiles + 3) / 4, k_splits);
    if (M <= 96) shared_rows_gemm_kernel<6, 1, EPI><<<blocks, 4 * WAVE, 0, stream>>>(p);
    else shared_rows_gemm_kernel<8, 1, EPI><<<blocks, 4 * WAVE, 0, stream>>>(p);
    return 0;
  }
  return ERR_UNSUPPORTED_SIZE;
}

// Sizes: 1 <= M <= 64, K a multiple of 32; with the NORM prologue the step's M normalized rows must fit
// 64 KiB of LDS beside the reduction area (16 rows of 1,024, 8 of 3,072).  EPI_SWIGLU wants N a multiple of 16.
// w_fragments: W is not row-major [N, K] but a copy in the order of the matrix-core fragments,
// [ceil(N / 16), K / 32, 4, 16, 8] with element [n, c, q, r, j] = W[16 n + r, 32 c + 8 q + j] (rows past N zero):
// what a wave asks for at once is then one run of 1 KiB instead of 64 bytes of each of 16 rows, which
// streams 15 to 25 % faster.  feature_tiles -1 or -2 (K >= 128, plain prologue, bfloat16 out): that
// many tiles a wave of the kernel whose waves share the step's rows through LDS.
extern "C" int mi_fused_gemm(int pro, int epi, const float* h_in, const void* delta0, const void* delta1,
                             float* h_out, const float* norm_w, float eps, const void* x, long x_ld,
                             const void* W, const float* bias, int M, int N, int K, void* out, long out_ld,
                             int out_f32, float out_scale, int conv_lo, int conv_hi, int conv_k,
                             const float* conv_w, const float* conv_b, void* conv_state, const int* slot_ids,
                             int feature_tiles, int w_fragments, const float* ssq_in, int ssq_blocks, int ssq_width,
                             float ssq_eps, int row_tiles, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !out) return ERR_BAD_ARGUMENT;
  if (ssq_in && (pro != PRO_PLAIN || ssq_blocks <= 0 || ssq_width <= 0)) return ERR_BAD_ARGUMENT;
  const bool shared_rows = feature_tiles < 0;       // -1, -2: that many tiles a wave of shared_rows_gemm_kernel
  if (shared_rows && (feature_tiles < -2 || pro != PRO_PLAIN || out_f32)) return ERR_BAD_ARGUMENT;
  if (row_tiles < 1 || row_tiles > 4 || (row_tiles > 1 && (shared_rows || pro != PRO_PLAIN || feature_tiles != 1)))
    return ERR_BAD_ARGUMENT;
  if (!shared_rows && feature_tiles != 1 && feature_tiles != 2 && feature_tiles != 4) return ERR_BAD_ARGUMENT;
  if (M > 64 || K % 32 != 0) return ERR_UNSUPPORTED_SIZE;
  if (shared_rows && K / 32 < SR_CHUNKS) return ERR_UNSUPPORTED_SIZE;
  if (pro == PRO_NORM && (!h_in || !norm_w || h_out == h_in)) return ERR_BAD_ARGUMENT;
  if (pro == PRO_PLAIN && (!x || x_ld < K || x_ld % 8 != 0)) return ERR_BAD_ARGUMENT;
  if (epi == EPI_SWIGLU && (N % 16 != 0 || out_f32)) return ERR_BAD_ARGUMENT;
  if (epi == EPI_CONV && (conv_lo < 0 || conv_hi > N || conv_hi <= conv_lo || conv_k < 1 || !conv_w ||
                          (conv_k > 1 && (!conv_state || !slot_ids)) || out_f32))
    return ERR_BAD_ARGUMENT;
  const int MT = (M + 15) / 16;
  if (pro != PRO_NORM && pro != PRO_PLAIN) return ERR_BAD_ARGUMENT;
  if (!shared_rows && fused_gemm_lds(MT, pro, K, M) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p = {};
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
  p.w_tiled = w_fragments ? 1 : 0;
  p.ssq_in = ssq_in;
  p.ssq_blocks = ssq_blocks;
  p.ssq_width = ssq_width;
  p.ssq_eps = ssq_eps;
  int code;
  if (shared_rows && epi != EPI_SWIGLU) {           // plain rows in bfloat16: the conv epilogue without a conv column
    if (epi == EPI_PLAIN) {
      p.conv_lo = p.conv_hi = 0;
      p.conv_k = 1;
    }
    code = launch_shared_rows_for<EPI_CONV>(M, p, stream, 1, -feature_tiles);
  } else if (shared_rows) code = launch_shared_rows_for<EPI_SWIGLU>(M, p, stream, 1, -feature_tiles);
  else code = launch_fused_gemm_rows(p, pro, epi, stream, 1, feature_tiles, row_tiles);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// The same product split over K for steps of many rows and few output features (a long K over 64
// workgroups leaves most of the GPU idle): `splits` rows of workgroups each take a run of K and write
// float32 partial sums into slab s of `partial` [splits, M, N] (the bias goes into slab 0).  The slabs
// are added up by whoever reads them: the residual add of the next norm.
extern "C" int mi_fused_gemm_split(const void* x, long x_ld, const void* W, const float* bias, int M, int N, int K,
                                   float* partial, int splits, int feature_tiles, int w_fragments,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !x || !partial || x_ld < K || x_ld % 8 != 0) return ERR_BAD_ARGUMENT;
  if (feature_tiles != 1 && feature_tiles != 2 && feature_tiles != 4) return ERR_BAD_ARGUMENT;
  if (M > 64 || K % 32 != 0 || splits < 1 || splits > 64 || K / 32 < splits) return ERR_UNSUPPORTED_SIZE;
  const int MT = (M + 15) / 16;
  if (fused_gemm_lds(MT, PRO_PLAIN, K, M) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p = {};
  p.x = (const bf16_t*)x;
  p.x_ld = x_ld;
  p.W = (const bf16_t*)W;
  p.bias = bias;
  p.M = M;
  p.N = N;
  p.K = K;
  p.out = partial;
  p.out_ld = N;
  p.out_f32 = 1;
  p.out_scale = 1.0f;
  p.w_tiled = w_fragments ? 1 : 0;
  const int code = launch_fused_gemm_rows(p, PRO_PLAIN, EPI_PLAIN, stream, splits, feature_tiles);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// The same slabs for steps of up to 128 rows through shared_rows_gemm_kernel: a workgroup's four waves own
// feature_tiles (1 or 2; 1 beyond 64 rows) tiles of 16 features each and share the step's rows through LDS.
// K >= 128.
extern "C" int mi_shared_rows_gemm_split(const void* x, long x_ld, const void* W, const float* bias, int M, int N,
                                         int K, float* partial, int splits, int feature_tiles, int w_fragments,
                                         hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !x || !partial || x_ld < K || x_ld % 8 != 0) return ERR_BAD_ARGUMENT;
  if (feature_tiles != 1 && feature_tiles != 2) return ERR_BAD_ARGUMENT;
  if (M > 128 || K % 32 != 0 || K / 32 < SR_CHUNKS || splits < 1 || splits > 64 || K / 32 < splits)
    return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p = {};
  p.x = (const bf16_t*)x;
  p.x_ld = x_ld;
  p.W = (const bf16_t*)W;
  p.bias = bias;
  p.M = M;
  p.N = N;
  p.K = K;
  p.out = partial;
  p.out_ld = N;
  p.out_f32 = 1;
  p.out_scale = 1.0f;
  p.w_tiled = w_fragments ? 1 : 0;
  const int code = launch_shared_rows_for<EPI_PLAIN>(M, p, stream, splits, feature_tiles);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// out[M, N] (bfloat16) = x[M, K] . W[N, K]^T + bias, where the first heads * head_dim columns of x are not read
// from x but merged from `partial`, the (maximum, normalizer, sums) that mi_mixer_decode (merge = 0) left per
// run of keys: [M, heads, runs, head_dim + 2], with the same runs, run_keys, page_size and window.  Every
// workgroup merges all of them again (a few hundred KB from the caches), which is cheaper than a launch of
// mixer_merge_kernel while the step is small.  M <= 16; the merged columns must fit LDS beside the sums.
// With res_h the result is not stored in `out` but added to the residual stream (the RESIDUAL epilogue, as in
// mi_fused_gemm_residual).
extern "C" int mi_fused_gemm_merge(const float* partial, const int* positions, int heads, int head_dim, int runs,
                                   int run_keys, int page_size, int window, const void* x, long x_ld, const void* W,
                                   const float* bias, int M, int N, int K, void* out, long out_ld, int w_fragments,
                                   float* res_h, void* res_hb, long res_hb_ld, const float* res_w, float* ssq_out,
                                   hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !x || !partial || !positions || x_ld < K || x_ld % 8 != 0)
    return ERR_BAD_ARGUMENT;
  if (res_h ? (!res_hb || !res_w || !ssq_out || res_hb_ld < N) : !out) return ERR_BAD_ARGUMENT;
  if (heads <= 0 || head_dim <= 0 || runs <= 0 || run_keys <= 0 || page_size <= 0 || window < 0) return ERR_BAD_ARGUMENT;
  const long merged = (long)heads * head_dim;
  if (M > 16 || K % 32 != 0 || head_dim % 8 != 0 || merged % 32 != 0 || merged > K) return ERR_UNSUPPORTED_SIZE;
  if (fused_gemm_lds(1, PRO_MERGE, K, M, (int)merged) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p = {};
  p.x = (const bf16_t*)x;
  p.x_ld = x_ld;
  p.W = (const bf16_t*)W;
  p.bias = bias;
  p.M = M;
  p.N = N;
  p.K = K;
  p.out = out;
  p.out_ld = out_ld;
  p.out_scale = 1.0f;
  p.w_tiled = w_fragments ? 1 : 0;
  p.partial = partial;
  p.positions = positions;
  p.merge_heads = heads;
  p.merge_dh = head_dim;
  p.merge_runs = runs;
  p.merge_run_keys = run_keys;
  p.merge_page = page_size;
  p.merge_window = window;
  p.res_h = res_h;
  p.res_hb = (bf16_t*)res_hb;
  p.res_hb_ld = res_hb_ld;
  p.res_w = res_w;
  p.ssq_out = ssq_out;
  const int code = launch_fused_gemm_rows(p, PRO_MERGE, res_h ? EPI_RESIDUAL : EPI_PLAIN, stream);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// h[M, N] += x[M, K] . W[N, K]^T + bias in float32, in place: a projection whose result joins the residual stream.
// Beside it, what the next norm's product needs without a pass of its own: hb[M, hb_ld] = bfloat16(h * next_w[n]),
// the new rows times that norm's weight, and ssq_out[ceil(N / 16), 16 ceil(M / 16)], the sums of squares of each
// new row over each workgroup's 16 features (mi_fused_gemm takes them as its row scale).  M <= 64.
extern "C" int mi_fused_gemm_residual(const void* x, long x_ld, const void* W, const float* bias, int M, int N, int K,
                                      float* res_h, void* res_hb, long res_hb_ld, const float* res_w, float* ssq_out,
                                      int w_fragments, int row_tiles, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || !W || !x || x_ld < K || x_ld % 8 != 0 || !res_h || !res_hb || !res_w || !ssq_out ||
      res_hb_ld < N)
    return ERR_BAD_ARGUMENT;
  if (M > 64 || K % 32 != 0) return ERR_UNSUPPORTED_SIZE;
  if (row_tiles < 1 || row_tiles > 4) return ERR_BAD_ARGUMENT;
  const int MT = (M + 15) / 16;
  if (fused_gemm_lds(MT, PRO_PLAIN, K, M) > 64 * 1024) return ERR_UNSUPPORTED_SIZE;
  FusedGemmParams p = {};
  p.x = (const bf16_t*)x;
  p.x_ld = x_ld;
  p.W = (const bf16_t*)W;
  p.bias = bias;
  p.M = M;
  p.N = N;
  p.K = K;
  p.out_scale = 1.0f;
  p.w_tiled = w_fragments ? 1 : 0;
  p.res_h = res_h;
  p.res_hb = (bf16_t*)res_hb;
  p.res_hb_ld = res_hb_ld;
  p.res_w = res_w;
  p.ssq_out = ssq_out;
  const int code = launch_fused_gemm_rows(p, PRO_PLAIN, EPI_RESIDUAL, stream, 1, 1, row_tiles);
  if (code != 0) return code;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// Whether mi_fused_gemm covers a shape (the host asks before it builds a fused path).
extern "C" int mi_fused_gemm_supported(int pro, int M, int K) {
  if (M <= 0 || M > 64 || K % 32 != 0) return 0;
  return fused_gemm_lds((M + 15) / 16, pro, K, M) <= 64 * 1024 ? 1 : 0;
}

// ---------------------------------------------------------------- mixer decode
#define MX_THREADS 512
#define MX_WAVES 8
#define MX_MAX_PAGES 132       // page ids of one run of keys (at most MX_SPLIT_MOST / 8 + 2)
#define MX_SPLIT_LEAST 256     // keys of one attention workgroup: between these two, see mi_mixer_split_keys
#define MX_SPLIT_MOST 1024
#define MX_WALK_BLOCKS 256      // attention workgroups from which on a workgroup walks over several runs
#define MX_SPLIT_BLOCKS 128    // attention workgroups a step should at least have before its runs grow
#define MX_SCAN_PER_THREAD 8
#define MX_FEW_BLOCKS 512       // state-space workgroups of a step up to which each takes one row per thread group

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
  int window;
  // state space
  int H, P, N, G, R, p_tiles, vector_scan, rows_per_thread, z_col, x_col, dt_col;
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
  // the context of a request is cut into runs of split_keys keys, one workgroup each; their
  // partial results [M, Hq, splits, DH + 2] = (maximum, normalizer, sums) are merged by mixer_merge_kernel
  int splits;
  int split_keys;
  float* partial;
};

// one dim of a rotated head: pairs (j, j + rotary_dim/2) of the first rotary_dim dims;
// cs holds cos (first half) and sin (second half) of the token's angles, rotary_dim/2 each
__device__ __forceinline__ float rotated_dim(const bf16_t* head, int dim, int rotary_dim, const float* cs) {
  const float x = (float)head[dim];
  if (dim >= rotary_dim) return x;
  const int half = rotary_dim / 2;
  const int j = dim < half ? dim : dim - half;
  const float c = cs[j], s = cs[half + j];
  return dim < half ? x * c - (float)head[dim + half] * s : x * c + (float)head[dim - half] * s;
}

// Latency matters more than bandwidth here (a request's K and V for one layer are about a
// megabyte): what a workgroup does is a chain of dependent memory round trips, so the context is
// cut into runs of split_keys keys, one workgroup per (token, kv head, run), each wave of which
// asks for all its keys at once (64 keys: two steps of attn_mfma.h in flight, the query heads of
// the kv head as the columns).  The waves merge through LDS and the workgroup leaves (maximum,
// normalizer, sums) per head; a small kernel merges the runs (a merge inside this kernel would
// need a device-wide fence, which costs more than the whole read).  The new token's rotated key
// and its value are written to their cache cell by the workgroup whose run holds it, before it
// reads, so the run reads them like any other key.
template <int DH>
__device__ void mixer_attention_block(const MixerParams& p, int block, int* pages_lds, float* cs,
                                      float* merge_lds) {
  const int G = p.Hq / p.Hkv;
  const int split = block % p.splits;
  const int kvh = (block / p.splits) % p.Hkv;
  const long token = block / (p.splits * p.Hkv);
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int qd = lane / 16;
  const int n = lane % 16;
  const bf16_t* row = p.u + token * p.u_ld;
  const int* table = p.block_tables + token * p.max_pages;
  const int half = p.rotary_dim / 2;

  // ---- everything that does not depend on the position is asked for at once, with no branch
  // between the loads (an index that is not needed is clamped to one that is valid): the query
  // heads, the new key and value, the cache cell, the rotation frequencies
  const bool rotate = p.inv_freq != nullptr;
  // (the position first: the page ids wait for it, the keys for them, and loads come back in the order they were
  // asked for; behind the query's rows, which the kernel before has just written on other dies, it would wait for them)
  const int pos = p.positions[token];
  const long cell = p.slot_mapping[token];
  mfma_bf16x8 q_own[DH / 32], q_pair[DH / 32];
  const bool has_head = n < G;
  const bf16_t* q_head = row + p.q_col + (kvh * G + (has_head ? n : 0)) * DH;
#pragma unroll
  for (int kk = 0; kk < DH / 32; ++kk) {
    const int own_dim = 32 * kk + 8 * qd;
    const int pair_dim = own_dim < p.rotary_dim ? (own_dim < half ? own_dim + half : own_dim - half) : own_dim;
    q_own[kk] = *reinterpret_cast<const mfma_bf16x8*>(q_head + own_dim);
    q_pair[kk] = *reinterpret_cast<const mfma_bf16x8*>(q_head + pair_dim);
  }
  const int k_dim = min(tid, DH - 1);
  const int k_pair_dim = k_dim < p.rotary_dim ? (k_dim < half ? k_dim + half : k_dim - half) : k_dim;
  const bf16_t* k_head = row + p.k_col + kvh * DH;
  const bf16_t k_raw_bits = k_head[k_dim];
  const bf16_t k_pair_bits = k_head[k_pair_dim];
  const bf16_t v_raw_bits = row[p.v_col + kvh * DH + k_dim];
  const float frequency = rotate ? p.inv_freq[min(tid, max(half, 1) - 1)] : 0.f;

  // ---- this workgroup's run of keys
  int first_key = 0;
  if (p.window > 0 && pos - p.window + 1 > 0) first_key = pos - p.window + 1;
  const int base_key = (first_key / p.page_size) * p.page_size;       // a page edge
  // the request's keys are cut into runs of split_keys; this workgroup takes the runs split, split + splits,
  // split + 2 splits, ... (a large step has fewer workgroups than runs: a workgroup that finds no keys costs
  // some 30 ns of a step's time, and a graph made for long contexts would launch hundreds of them)
  const int runs = (pos - base_key) / p.split_keys + 1;
  if (split >= runs) return;                                           // nothing of this request here
  const bool writer = (runs - 1) % p.splits == split;                  // the workgroup that holds the new token
  auto stage_pages = [&](int run) {
    const int lo = base_key + run * p.split_keys;
    const int hi = min(lo + p.split_keys, pos + 1);
    const int first_page = lo / p.page_size;
    const int last_page = (hi - 1) / p.page_size;
    for (int t = tid; t <= last_page - first_page; t += MX_THREADS) pages_lds[t] = table[first_page + t];
  };
  stage_pages(split);
  const float k_raw = (float)k_raw_bits, k_raw_pair = (float)k_pair_bits, v_raw = (float)v_raw_bits;
  if (rotate) {
    const float position = (float)pos;
    if (tid < half) {
      const float angle = position * frequency;
      cs[tid] = cosf(angle);
      cs[half + tid] = sinf(angle);
    }
    for (int j = tid + MX_THREADS; j < half; j += MX_THREADS) {      // head sizes beyond the workgroup: none today
      const float angle = position * p.inv_freq[j];
      cs[j] = cosf(angle);
      cs[half + j] = sinf(angle);
    }
  }
  __syncthreads();

  // the new token's key (rotated) and value go to their cache cell
  if (writer && tid < DH) {
    float k = k_raw;
    if (rotate && tid < p.rotary_dim) {
      const int j = tid < half ? tid : tid - half;
      k = tid < half ? k_raw * cs[j] - k_raw_pair * cs[half + j] : k_raw * cs[j] + k_raw_pair * cs[half + j];
    }
    const long page = cell / p.page_size;
    const int offset = (int)(cell - page * p.page_size);
    p.k_base[page * p.page_stride + ((long)kvh * p.page_size + offset) * DH + tid] = (bf16_t)k;
    p.v_base[page * p.page_stride + ((long)kvh * DH + tid) * p.page_size + offset] = (bf16_t)v_raw;
  }
  // q: rotated in float32, rounded to bfloat16 as when it is stored
  mfma_bf16x8 q_frag[1][DH / 32];
#pragma unroll
  for (int kk = 0; kk < DH / 32; ++kk) {
    const int own_dim = 32 * kk + 8 * qd;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float value = (float)q_own[kk][j];
      if (rotate && own_dim < p.rotary_dim) {
        const int dim = own_dim + j;
        const int f = dim < half ? dim : dim - half;
        value = dim < half ? value * cs[f] - (float)q_pair[kk][j] * cs[half + f]
                           : value * cs[f] + (float)q_pair[kk][j] * cs[half + f];
      }
      q_frag[0][kk][j] = has_head ? (bf16_t)value : (bf16_t)0.f;
    }
  }
  __threadfence_block();
  __syncthreads();

  // ---- this wave's share of each run
  int span = (p.split_keys + MX_WAVES - 1) / MX_WAVES;
  span = ((span + 31) / 32) * 32;
  AttnAccumulator<DH, 1> acc;
  acc.clear();
  for (int run = split; run < runs; run += p.splits) {
    if (run != split) {
      __syncthreads();                                                 // the page ids of the run before are read
      stage_pages(run);
      __syncthreads();
    }
    const int run_lo = base_key + run * p.split_keys;
    const int run_hi = min(run_lo + p.split_keys, pos + 1);
    const int wave_lo = run_lo + wave * span;
    const int wave_hi = min(wave_lo + span, run_hi);
    if (wave_lo < run_hi) {
      AttnCache cache;
      cache.k_base = p.k_base;
      cache.v_base = p.v_base;
      cache.page_stride = p.page_stride;
      cache.page_size = p.page_size;
      cache.kvh = kvh;
      cache.pages = pages_lds;
      cache.base_page = run_lo / p.page_size;
      const int col_pos[1] = {has_head ? pos : -1};
      attend_keys<DH, 1, 2>(acc, q_frag, col_pos, p.window, p.scale, wave_lo, wave_hi, cache);
    }
  }

  // ---- merge the waves: merge_lds[wave][head] = {m, l, o[DH]}
  const float l = attn_normalizer<DH, 1>(acc, 0);
  if (has_head) {
    float* mine = merge_lds + (long)(wave * G + n) * (DH + 2);
    if (qd == 0) {
      mine[0] = acc.m[0];
      mine[1] = l;
    }
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) mine[2 + 16 * dt + 4 * qd + i] = acc.o[0][dt][i];
  }
  __syncthreads();
  for (int index = tid; index < G * DH; index += MX_THREADS) {
    const int g = index / DH;
    const int dim = index - g * DH;
    float maximum = -INFINITY;
#pragma unroll
    for (int w = 0; w < MX_WAVES; ++w) maximum = fmaxf(maximum, merge_lds[(long)(w * G + g) * (DH + 2)]);
    float denominator = 0.f, sum = 0.f;
#pragma unroll
    for (int w = 0; w < MX_WAVES; ++w) {
      const float* theirs = merge_lds + (long)(w * G + g) * (DH + 2);
      const float weight = __builtin_amdgcn_exp2f(theirs[0] - maximum);      // 0 for a wave without keys (m = -inf); maxima are in units of log2
      denominator += weight * theirs[1];
      sum += weight * theirs[2 + dim];
    }
    if (p.splits == 1) {             // the only workgroup of this token and kv head: nothing is left to merge
      p.attn_out[token * p.out_ld + (long)(kvh * G + g) * DH + dim] = (bf16_t)(sum / denominator);
      continue;
    }
    float* mine = p.partial + ((token * p.Hq + kvh * G + g) * p.splits + split) * (long)(DH + 2);
    if (dim == 0) {
      mine[0] = maximum;
      mine[1] = denominator;
    }
    mine[2 + dim] = sum;
  }
}

// out[token, head, :] = sum_s exp(m_s - m) o_s / sum_s exp(m_s - m) l_s over the runs that hold keys.
// Eight runs are asked for at once, before it is known how many hold keys (the position is on
// its way too); what a run without keys left in its place is read and not used.
__global__ void mixer_merge_kernel(MixerParams p, int dh) {
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int dim = min((int)threadIdx.x, dh - 1);
  const float* runs = p.partial + (token * p.Hq + head) * p.splits * (long)(dh + 2);
  const int pos = p.positions[token];
  float maximum = -INFINITY, denominator = 0.f, sum = 0.f;
  int used = p.splits;
  for (int s0 = 0; s0 < used; s0 += MERGE_AT_ONCE) {
    float m_s[MERGE_AT_ONCE], l_s[MERGE_AT_ONCE], o_s[MERGE_AT_ONCE];
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j) {
      const float* run = runs + (long)min(s0 + j, p.splits - 1) * (dh + 2);
      m_s[j] = run[0];
      l_s[j] = run[1];
      o_s[j] = run[2 + dim];
    }
    if (s0 == 0) {
      int first_key = 0;
      if (p.window > 0 && pos - p.window + 1 > 0) first_key = pos - p.window + 1;
      const int base_key = (first_key / p.page_size) * p.page_size;
      used = min(p.splits, (pos - base_key) / p.split_keys + 1);
    }
#pragma unroll
    for (int j = 0; j < MERGE_AT_ONCE; ++j) {
      if (s0 + j < used) {
        const float larger = fmaxf(maximum, m_s[j]);
        const float keep = __builtin_amdgcn_exp2f(maximum - larger);        // 0 the first time (maximum = -inf); units of log2
        const float weight = __builtin_amdgcn_exp2f(m_s[j] - larger);
        denominator = denominator * keep + weight * l_s[j];
        sum = sum * keep + weight * o_s[j];
        maximum = larger;
      }
    }
  }
  if ((int)threadIdx.x < dh) p.attn_out[token * p.out_ld + (long)head * dh + dim] = (bf16_t)(sum / denominator);
}

// One step of the selective scan for (token, head, tile of state rows); see ssm_scan_kernel.
// A state row of N floats is shared by R lanes.  When N is 8*R (VECTOR) each lane owns 8
// consecutive elements: two 16-byte state loads and one 16-byte load each of B and C.
template <bool VECTOR, int RPT>
__device__ void mixer_ssm_block(const MixerParams& p, int block) {
  const int tile = block % p.p_tiles;
  const int head = (block / p.p_tiles) % p.H;
  const long token = block / (p.p_tiles * p.H);
  const int R = p.R;
  const int rows_per_round = MX_THREADS / R;
  const int row_in_round = threadIdx.x / R;
  const int r = threadIdx.x - row_in_round * R;
  const int group = head / (p.H / p.G);
  const int N = p.N;
  const bf16_t* row = p.u + token * p.u_ld;
  const bf16_t* b_row = row + p.x_col + p.H * p.P + group * N;
  const bf16_t* c_row = b_row + p.G * N;
  // a thread owns 8 state elements of RPT rows (large batches: more bytes in flight per thread and
  // fewer workgroups, each of which first waits for its slot id).  Every load of the step is asked for
  // before the first is used (the state first: it comes from furthest away), with no branch between
  // them; a row past P reads row 0 and is dropped
  int pi[RPT];
  bool active[RPT];
  float* s_row[RPT];
  const long slot_base = ((long)p.slot_ids[token] * p.H + head) * p.P;
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    pi[j] = (tile * RPT + j) * rows_per_round + row_in_round;
    active[j] = pi[j] < p.P;
    s_row[j] = p.ssm_state + (slot_base + (active[j] ? pi[j] : 0)) * N;
  }
  floatx4 s0[RPT], s1[RPT];
  bf16x8_t b, c;
  if (VECTOR) {
#pragma unroll
    for (int j = 0; j < RPT; ++j) {
      s0[j] = *reinterpret_cast<const floatx4*>(s_row[j] + r * 8);
      s1[j] = *reinterpret_cast<const floatx4*>(s_row[j] + r * 8 + 4);
    }
    b = *reinterpret_cast<const bf16x8_t*>(b_row + r * 8);
    c = *reinterpret_cast<const bf16x8_t*>(c_row + r * 8);
  }
  const bf16_t dt_bits = row[p.dt_col + head];
  bf16_t x_bits[RPT], z_bits[RPT];
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const long column = (long)head * p.P + (active[j] ? pi[j] : 0);
    x_bits[j] = row[p.x_col + column];
    z_bits[j] = row[p.z_col + column];
  }
  const float delta = softplus_f((float)dt_bits + p.dt_bias[head]);
  const float decay = expf(delta * p.A[head]);
  const float skip = p.D[head];
#pragma unroll
  for (int j = 0; j < RPT; ++j) {
    const long column = (long)head * p.P + (active[j] ? pi[j] : 0);
    const float x = active[j] ? (float)x_bits[j] : 0.f;
    const float dx = delta * x;
    float partial = 0.f;
    if (VECTOR) {
      if (active[j]) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          s0[j][i] = decay * s0[j][i] + dx * (float)b[i];
          s1[j][i] = decay * s1[j][i] + dx * (float)b[4 + i];
          partial += s0[j][i] * (float)c[i];
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) partial += s1[j][i] * (float)c[4 + i];
        *reinterpret_cast<floatx4*>(s_row[j] + r * 8) = s0[j];
        *reinterpret_cast<floatx4*>(s_row[j] + r * 8 + 4) = s1[j];
      }
    } else {
#pragma unroll
      for (int i = 0; i < MX_SCAN_PER_THREAD; ++i) {
        const int n = r + i * R;
        if (active[j] && n < N) {
          const float next = decay * s_row[j][n] + dx * (float)b_row[n];
          s_row[j][n] = next;
          partial += next * (float)c_row[n];
        }
      }
    }
    for (int offset = R / 2; offset > 0; offset >>= 1) partial += __shfl_xor(partial, offset, WAVE);
    if (active[j] && r == 0) {
      const float y = partial + skip * x;
      if (p.ssm_y) p.ssm_y[token * (long)(p.H * p.P) + column] = y;
      else p.ssm_out[token * p.out_ld + column] = (bf16_t)(y * silu_f((float)z_bits[j]));
    }
  }
}

template <int DH>
__global__ void __launch_bounds__(MX_THREADS) mixer_decode_kernel(MixerParams p) {
  __shared__ int pages_lds[MX_MAX_PAGES];
  __shared__ float cs[DH];
  __shared__ float merge_lds[MX_WAVES * 8 * (DH + 2)];
  if ((int)blockIdx.x < p.attention_blocks)
    mixer_attention_block<DH>(p, blockIdx.x, pages_lds, cs, merge_lds);
  else if (!p.vector_scan)
    mixer_ssm_block<false, 1>(p, blockIdx.x - p.attention_blocks);
  else if (p.rows_per_thread == 1)
    mixer_ssm_block<true, 1>(p, blockIdx.x - p.attention_blocks);
  else if (p.rows_per_thread == 2)
    mixer_ssm_block<true, 2>(p, blockIdx.x - p.attention_blocks);
  else if (DH == 64 || p.rows_per_thread == 4)         // eight rows cost the 64-wide kernel a wave per SIMD
    mixer_ssm_block<true, 4>(p, blockIdx.x - p.attention_blocks);
  else
    mixer_ssm_block<true, 8>(p, blockIdx.x - p.attention_blocks);
}

// Keys of one attention workgroup (a run).  Long runs pay the start of a workgroup (position, page ids,
// then keys: three round trips) and the merge of the runs less often; short runs give a small step more
// workgroups, and a request whose context ends just behind a run's edge pays a whole workgroup for a few
// keys.  Measured on one MI355X (mixer + merge of a layer, head size 64, 2 kv heads; runs of
// 256 / 512 / 1,024 keys; contexts inside graphs made for 4,096 and 8,192 keys): 1 token at 2,100 keys
// 11.3 / 12.0 / 15.0 us; 8 tokens at 2,100 keys 15.1 / 14.0 / 16.6, at 6,000 keys 20.3 / 17.2 / 17.8;
// 64 tokens at 2,100 keys 61.0 / 56.0 / 52.0, at 6,000 keys 100 / 85 / 80.  So: the longest run that still
// leaves MX_SPLIT_BLOCKS workgroups (up to 512 keys for steps of up to 16 tokens, 1,024 beyond), and never
// more than 16 runs for a request.  `span`: the most keys a request of the step can have.
extern "C" int mi_mixer_split_keys(int M, int Hkv, int page_size, long span) {
  if (M <= 0 || Hkv <= 0 || page_size <= 0 || span <= 0) return 0;
  long split = MX_SPLIT_LEAST;
  for (long candidate = M <= 16 ? MX_SPLIT_MOST / 2 : MX_SPLIT_MOST; candidate > MX_SPLIT_LEAST; candidate /= 2)
    if ((long)Hkv * M * ((span + candidate - 1) / candidate) >= MX_SPLIT_BLOCKS) {
      split = candidate;
      break;
    }
  while (split < MX_SPLIT_MOST && span > 16 * split) split *= 2;
  if (split < page_size) split = page_size;
  return (int)((split / page_size) * page_size);          // whole pages
}

// The runs of keys of a step, as mi_mixer_decode cuts them: keys of a run and workgroups (partial results) per
// (token, kv head): one per run while the step is small, fewer (each walks over several runs) once the step has
// MX_WALK_BLOCKS of them anyway.  `span`: the most keys a request of the step can have.
extern "C" int mi_mixer_runs(int M, int Hkv, int page_size, long span, int* run_keys, int* runs) {
  const int keys = mi_mixer_split_keys(M, Hkv, page_size, span);
  if (keys <= 0 || !run_keys || !runs) return ERR_BAD_ARGUMENT;
  const long whole = (span + keys - 1) / keys;
  *run_keys = keys;
  *runs = (int)min(whole, max(1L, (MX_WALK_BLOCKS + (long)Hkv * M - 1) / ((long)Hkv * M)));
  return 0;
}

// merge = 0: the attended heads are not written; `partial` is left for mi_fused_gemm_merge.  (When a token and
// kv head have one workgroup, mi_mixer_runs says runs = 1, there is nothing to merge: that workgroup writes the
// attended heads itself, whatever `merge` says, and no merge kernel is launched.)
extern "C" int mi_mixer_decode(const void* u, long u_ld, int M, int Hq, int Hkv, int dh, int q_col, int k_col,
                               int v_col, const float* inv_freq, int rotary_dim, void* k_base, void* v_base,
                               long page_stride, int page_size, const int* block_tables, int max_pages,
                               const int* positions, const int* slot_mapping, float scale, int window,
                               int max_seq_len, int H, int P, int N, int G, int z_col, int x_col, int dt_col, const float* dt_bias,
                               const float* A, const float* D, float* ssm_state, const int* slot_ids,
                               void* attn_out, void* ssm_out, float* ssm_y, long out_ld, float* partial,
                               long partial_floats, int merge, hipStream_t stream) {
  if (M <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || H <= 0 || P <= 0 || N <= 0 || G <= 0 || H % G != 0)
    return ERR_BAD_ARGUMENT;
  const int group = Hq / Hkv;
  const long span = window > 0 ? (long)window + page_size : (long)max_seq_len;
  if ((dh != 64 && dh != 128) || group > 8 || page_size % 8 != 0 || page_size > MX_SPLIT_LEAST * 2 || max_seq_len <= 0 ||
      N > WAVE * MX_SCAN_PER_THREAD ||
      u_ld % 8 != 0 || q_col % 8 != 0 || rotary_dim > dh || rotary_dim % 16 != 0)
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
  p.H = H;
  p.P = P;
  p.N = N;
  p.G = G;
  // a state row is shared by R lanes: N/8 of them with 8 consecutive elements each when N is
  // 8 times a power of two (and the rows of B and C are 16-byte aligned), else up to 64 with
  // strided elements
  int R = 1;
  const bool vector_scan = N % 8 == 0 && ((N / 8) & (N / 8 - 1)) == 0 && N / 8 <= WAVE &&
                           (x_col + H * P) % 8 == 0;
  if (vector_scan) {
    R = N / 8;
  } else {
    while (R < N && R < WAVE) R <<= 1;
  }
  p.R = R;
  p.vector_scan = vector_scan ? 1 : 0;
  // rows of a head per workgroup: one per thread group while the step has few workgroups (they hide each
  // other's latency); more from then on.  The state-space workgroups run at the register count of the
  // attention ones (two to four waves a SIMD), so what a large step needs is bytes in flight per thread;
  // a launch of their own at full occupancy was measured slower than that.
  int rows_per_block = MX_THREADS / R;
  p.rows_per_thread = 1;
  const int most_rows = dh == 128 ? 8 : 4;
  while (vector_scan && p.rows_per_thread < most_rows && rows_per_block < P &&
         (long)M * H * ((P + rows_per_block - 1) / rows_per_block) > MX_FEW_BLOCKS) {
    p.rows_per_thread *= 2;
    rows_per_block *= 2;
  }
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
  if (mi_mixer_runs(M, Hkv, page_size, span, &p.split_keys, &p.splits) != 0) return ERR_UNSUPPORTED_SIZE;
  if ((long)Hkv * M * p.splits > 0x3fffffffL || M > 65535 || Hq > 65535) return ERR_UNSUPPORTED_SIZE;
  if (!partial || partial_floats < (long)M * Hq * p.splits * (dh + 2)) return ERR_BAD_ARGUMENT;
  p.partial = partial;
  p.attention_blocks = Hkv * M * p.splits;
  const long total = (long)p.attention_blocks + (long)p.p_tiles * H * M;
  if (total > 0x7fffffffL) return ERR_UNSUPPORTED_SIZE;
  if (dh == 64) mixer_decode_kernel<64><<<(unsigned)total, MX_THREADS, 0, stream>>>(p);
  else mixer_decode_kernel<128><<<(unsigned)total, MX_THREADS, 0, stream>>>(p);
  RETURN_IF_LAUNCH_FAILED();
  if (!merge || p.splits == 1) return 0;
  const dim3 merge_grid(M, Hq);
  mixer_merge_kernel<<<merge_grid, dh, 0, stream>>>(p, dh);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
