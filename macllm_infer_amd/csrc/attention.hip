// Rotary position encoding fused with the write of K and V into cache pages, and
// attention over the paged cache.
//
// Cache layout of one paged group: [page, layer, 2 (K,V), kv_head, page_size*head_dim].
// Inside a page, K of one kv head is [token, dim] and V is transposed, [dim, token]: the
// value product contracts over tokens, and a matrix-core operand wants its contraction index
// contiguous.  Entry points get the base pointers of one layer's K and V inside page 0 and
// the stride between pages:
//   K(page, kvh, off, i) = k_base + page*page_stride + (kvh*page_size + off)*dh + i
//   V(page, kvh, off, i) = v_base + page*page_stride + (kvh*dh + i)*page_size + off
// (The reference pages its cache the same way, K and V both token-major:
// crates/macllm-kv/src/cache.rs:558-566, crates/macllm-kernels/src/metal/paged_decode.metal:109-113.)
#include "common.h"
#include <type_traits>

// ---------------------------------------------------------------- rope + cache write
// For token t at absolute position p:
//   q[t, h, :] is rotated in place; k[t, h, :] is rotated and stored; v[t, h, :] is stored.
//   Rotation (half-split, first rotary_dim dims): angle = (float)p * inv_freq[j];
//   out[j] = x[j] cos - x[j+half] sin;  out[j+half] = x[j+half] cos + x[j] sin.
//   (reference: src/decoder.rs:186-195, 226-229; K is cached after rotation, :953-962)
// slot_mapping[t] = page*page_size + offset of the token's cache cell; null = nothing is stored.
template <typename T>
__global__ void rope_kv_store_kernel(T* __restrict__ qkv, long ld, int Hq, int Hkv, int dh,
                                     const int* __restrict__ positions, const float* __restrict__ inv_freq,
                                     int rotary_dim, const int* __restrict__ slot_mapping,
                                     T* __restrict__ k_base, T* __restrict__ v_base, long page_stride,
                                     int page_size) {
  const long token = blockIdx.x;
  T* row = qkv + token * ld;
  const float position = (float)positions[token];
  const int half = rotary_dim / 2;
  long cell = -1;
  long page = 0;
  int offset = 0;
  if (slot_mapping) {
    cell = slot_mapping[token];
    page = cell / page_size;
    offset = (int)(cell - page * page_size);
  }
  // q heads then k heads: (head, pair) items
  const int rotary_heads = Hq + Hkv;
  const int pairs = rotary_heads * (dh / 2);   // items cover dh/2 "columns": rotated pairs and pass-through pairs
  for (int item = threadIdx.x; item < pairs; item += blockDim.x) {
    const int head = item / (dh / 2);
    const int j = item - head * (dh / 2);
    T* x = row + (long)head * dh;
    // column j pairs with j+half when j < half; columns >= rotary_dim pass through.
    // Enumerate so that every element of the head is visited exactly once:
    //   j in [0, half): rotated pair (j, j+half)
    //   j in [half, dh/2): pass-through elements (rotary_dim + 2*(j-half)) and the next one
    float a, b;
    int ia, ib;
    if (j < half) {
      ia = j;
      ib = j + half;
      const float x0 = to_float(x[ia]);
      const float x1 = to_float(x[ib]);
      float s = 0.f, c = 1.f;
      if (inv_freq) {
        const float angle = position * inv_freq[j];
        s = sinf(angle);
        c = cosf(angle);
      }
      a = x0 * c - x1 * s;
      b = x1 * c + x0 * s;
    } else {
      ia = rotary_dim + 2 * (j - half);
      ib = ia + 1;
      a = to_float(x[ia]);
      b = to_float(x[ib]);
    }
    if (head < Hq) {
      x[ia] = from_float<T>(a);
      x[ib] = from_float<T>(b);
    } else if (cell >= 0) {
      const int kvh = head - Hq;
      T* dst = k_base + page * page_stride + ((long)kvh * page_size + offset) * dh;
      dst[ia] = from_float<T>(a);
      dst[ib] = from_float<T>(b);
    }
  }
  if (cell >= 0) {
    const T* v = row + (long)(Hq + Hkv) * dh;
    for (int item = threadIdx.x; item < Hkv * dh; item += blockDim.x) {
      const int kvh = item / dh;
      const int i = item - kvh * dh;
      v_base[page * page_stride + ((long)kvh * dh + i) * page_size + offset] = v[item];
    }
  }
}

extern "C" int mi_rope_kv_store(void* qkv, int dtype, long ld, int T, int Hq, int Hkv, int dh,
                                const int* positions, const float* inv_freq, int rotary_dim,
                                const int* slot_mapping, void* k_base, void* v_base, long page_stride,
                                int page_size, hipStream_t stream) {
  if (T <= 0 || Hq <= 0 || Hkv <= 0 || dh <= 0 || (dh & 1)) return ERR_BAD_ARGUMENT;
  if (rotary_dim < 0 || rotary_dim > dh || (rotary_dim & 1)) return ERR_BAD_ARGUMENT;
  if (ld < (long)(Hq + 2 * Hkv) * dh) return ERR_BAD_ARGUMENT;
  if (slot_mapping && (!k_base || !v_base || page_size <= 0)) return ERR_BAD_ARGUMENT;
  if (!inv_freq) rotary_dim = 0;
  if (dtype == DT_F32)
    rope_kv_store_kernel<float><<<T, 256, 0, stream>>>((float*)qkv, ld, Hq, Hkv, dh, positions, inv_freq,
                                                        rotary_dim, slot_mapping, (float*)k_base,
                                                        (float*)v_base, page_stride, page_size);
  else if (dtype == DT_BF16)
    rope_kv_store_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)qkv, ld, Hq, Hkv, dh, positions, inv_freq,
                                                         rotary_dim, slot_mapping, (bf16_t*)k_base,
                                                         (bf16_t*)v_base, page_stride, page_size);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- paged attention, any size
// Works for any head_dim <= 256, any page size, any group size, float32 and bfloat16; the float32 path of
// the whole model uses it for prompts and for decoding alike.
//   s = q.k * scale;  visible keys: position <= query position, and
//   query - key < window when window > 0 (reference: src/decoder.rs:4515-4532);
//   softmax in float32 (reference: src/decoder.rs:4665-4667).
// `slopes` (optional, float32 per query head): a position encoding that is a bias on the scores,
//   s -= slopes[head] * (query position - key position)   (no counterpart in the reference).
// The keys are cut into runs of PA_RUN by their absolute position.  One workgroup per (token, query head,
// run): each of its four waves takes 64 keys of the run (lane i scores key i with a full dot product over
// dh from its own cache row; for the value product lane i owns output dims i, i + 64, ...), keeps
// (maximum, normalizer, sums) in float32, the waves are merged through LDS in their order and the workgroup
// leaves one partial result; a second kernel merges the runs in ascending order (the (maximum, normalizer,
// accumulator) merge the reference does across simdgroups, crates/macllm-kernels/src/metal/paged_decode.metal:145-183).
// Which keys meet in a wave, and the order of every sum, depend on the query's position alone: a token's
// result is bit for bit the same whatever else the step holds and however long the longest context is.
#define ATT_MAX_DH 256
#define PA_RUN 256
#define PA_WAVES (PA_RUN / WAVE)

template <typename T, bool FAST_EXP>
__global__ void __launch_bounds__(PA_RUN)
paged_attention_kernel(const T* __restrict__ q, long q_ld, int Hq, int Hkv, int dh,
                       const T* __restrict__ k_base, const T* __restrict__ v_base, long page_stride,
                       int page_size, const int* __restrict__ block_tables, int max_pages,
                       const int* __restrict__ lane_of_token, const int* __restrict__ positions, float scale,
                       int window, const float* __restrict__ slopes, int runs, float* __restrict__ partial) {
  typedef T vec4 __attribute__((ext_vector_type(4)));
  __shared__ __align__(16) float q_shared[ATT_MAX_DH];
  __shared__ float p_shared[PA_WAVES][WAVE];
  __shared__ long row_shared[PA_WAVES][WAVE];     // base of the key's (page, kv head) block
  __shared__ int offset_shared[PA_WAVES][WAVE];   // the key's place inside its page
  __shared__ float wave_ml[PA_WAVES][2];
  __shared__ float wave_o[PA_WAVES][ATT_MAX_DH];
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int run = blockIdx.z;
  const int query_position = positions[token];
  int first_key = 0;
  if (window > 0 && query_position - window + 1 > 0) first_key = query_position - window + 1;
  if ((run + 1) * PA_RUN <= first_key || run * PA_RUN > query_position) return;   // no key of this run is visible
  const int kvh = head / (Hq / Hkv);
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int* table = block_tables + (long)lane_of_token[token] * max_pages;
  const T* q_row = q + token * q_ld + (long)head * dh;
  for (int i = tid; i < dh; i += PA_RUN) q_shared[i] = to_float(q_row[i]);
  __syncthreads();

  const int key = run * PA_RUN + wave * WAVE + lane;
  const bool visible = key >= first_key && key <= query_position;
  float score = -INFINITY;
  long row_offset = 0;
  int offset = 0;
  if (visible) {
    const int page = table[key / page_size];
    offset = key % page_size;
    row_offset = (long)page * page_stride + (long)kvh * page_size * dh;
    const T* k_row = k_base + row_offset + (long)offset * dh;
    float dot = 0.f;
    if (dh % 4 == 0 && page_stride % 4 == 0 && ((unsigned long long)k_base % (4 * sizeof(T))) == 0) {
      for (int i = 0; i < dh; i += 4) {
        const vec4 piece = *reinterpret_cast<const vec4*>(k_row + i);
#pragma unroll
        for (int j = 0; j < 4; ++j) dot = fmaf(q_shared[i + j], to_float<T>(piece[j]), dot);
      }
    } else {
      for (int i = 0; i < dh; ++i) dot = fmaf(q_shared[i], to_float(k_row[i]), dot);
    }
    score = dot * scale;
    if (slopes) score = fmaf(-slopes[head], (float)(query_position - key), score);
  }
  const float maximum = wave_max(score);                    // -inf for a wave without visible keys
  const float p = visible ? (FAST_EXP ? __expf(score - maximum) : expf(score - maximum)) : 0.f;
  p_shared[wave][lane] = p;
  row_shared[wave][lane] = row_offset;
  offset_shared[wave][lane] = offset;
  __syncthreads();
  const int wave_first = run * PA_RUN + wave * WAVE;
  const int from = min(WAVE, max(0, first_key - wave_first));
  const int to = min(WAVE, max(0, query_position - wave_first + 1));
  if (lane == 0) {
    // the normalizer: the probabilities added up in the order of their keys (a sum whose order the keys fix,
    // not the lanes: the tiled kernel below forms the same sum without a pass over the wave)
    float normalizer = 0.f;
    for (int j = from; j < to; ++j) normalizer += p_shared[wave][j];
    wave_ml[wave][0] = maximum;
    wave_ml[wave][1] = normalizer;
  }
#pragma unroll
  for (int i = 0; i < ATT_MAX_DH / WAVE; ++i) {
    const int dim = lane + i * WAVE;
    if (dim < dh) {
      // sixteen values asked for at once, then added in the order of their keys (one at a time, each load would
      // wait for the one before: 64 round trips a wave); a key past the last reads the last again and is not added
      float sum = 0.f;
      for (int j0 = from; j0 < to; j0 += 16) {
        float values[16];
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const int j = min(j0 + u, to - 1);
          values[u] = to_float(v_base[row_shared[wave][j] + (long)dim * page_size + offset_shared[wave][j]]);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 16; ++u) {
          const float added = fmaf(p_shared[wave][min(j0 + u, WAVE - 1)], values[u], sum);
          sum = j0 + u < to ? added : sum;
        }
      }
      wave_o[wave][dim] = sum;
    }
  }
  __syncthreads();
  // the waves in their order; a wave without keys has the weight exp(-inf) = 0
  float best = wave_ml[0][0];
#pragma unroll
  for (int w = 1; w < PA_WAVES; ++w) best = fmaxf(best, wave_ml[w][0]);
  float* mine = partial + ((token * Hq + head) * runs + run) * (long)(dh + 2);
  float weight[PA_WAVES];
  float denominator = 0.f;
#pragma unroll
  for (int w = 0; w < PA_WAVES; ++w) {
    weight[w] = FAST_EXP ? __expf(wave_ml[w][0] - best) : expf(wave_ml[w][0] - best);
    denominator = fmaf(weight[w], wave_ml[w][1], denominator);
  }
  if (tid == 0) {
    mine[0] = best;
    mine[1] = denominator;
  }
  for (int dim = tid; dim < dh; dim += PA_RUN) {
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < PA_WAVES; ++w) sum = fmaf(weight[w], wave_o[w][dim], sum);
    mine[2 + dim] = sum;
  }
}

// The same partial results for steps whose lanes hold several tokens, from a workgroup that takes PT_QUERIES
// consecutive tokens of one lane, one query head and one run of PA_RUN keys: the run's keys and values go through
// LDS once for all of its queries, 64 keys at a time (the per-token kernel above fetches them once a token: a
// prompt of 2,048 tokens reads every key a thousand times).  A query's scores, softmax and sums are the per-token
// kernel's, operation for operation: 64 keys a wave-sized group in the order of their positions, lane i scoring
// key i with a dot product in ascending dims, the group's maximum and normalizer over the wave, lane d summing
// dim d in ascending keys, the four groups of a run weighted and added in their order.  So a position's result is
// the same bits from either kernel: whole prompts, portions and single tokens agree.
// Wave w takes the queries w, w + 4, ... of the tile.
// The largest value of a wave, in every lane: shifts within the rows of 16 lanes, then the last lane of a row
// to the row behind it, then the last lane of the lower half to the upper half (the data-parallel primitives of
// this GPU family; a maximum does not depend on the order it is taken in, so this is wave_max without six trips
// through the LDS crossbar).
template <int CONTROL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_minus_infinity(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, -INFINITY), __builtin_bit_cast(int, x),
                                                               CONTROL, ROW_MASK, 0xf, false));
}

__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, dpp_or_minus_infinity<0x111, 0xf>(v));      // row_shr:1
  v = fmaxf(v, dpp_or_minus_infinity<0x112, 0xf>(v));      // row_shr:2
  v = fmaxf(v, dpp_or_minus_infinity<0x114, 0xf>(v));      // row_shr:4
  v = fmaxf(v, dpp_or_minus_infinity<0x118, 0xf>(v));      // row_shr:8: lane 15 of each row holds the row's maximum
  v = fmaxf(v, dpp_or_minus_infinity<0x142, 0xa>(v));      // row_bcast:15 into rows 1 and 3
  v = fmaxf(v, dpp_or_minus_infinity<0x143, 0xc>(v));      // row_bcast:31 into rows 2 and 3: lane 63 holds the wave's maximum
  return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}

#define PT_QUERIES 16
#define PT_PER_WAVE (PT_QUERIES / PA_WAVES)
#define PT_PAD 4

// DIMS: dims of a head a lane sums (1, 2 or 4: the head size in units of 64, rounded up)
template <typename T, bool FAST_EXP, int DIMS>
__global__ void __launch_bounds__(PA_RUN)
paged_attention_tile_kernel(const T* __restrict__ q, long q_ld, int Hq, int Hkv, int dh,
                            const T* __restrict__ k_base, const T* __restrict__ v_base, long page_stride,
                            int page_size, const int* __restrict__ block_tables, int max_pages,
                            const int* __restrict__ query_tiles, int tile_tokens, const int* __restrict__ cu_seqlens,
                            const int* __restrict__ positions, float scale, int window,
                            const float* __restrict__ slopes, int runs, float* __restrict__ partial) {
  typedef T vec4 __attribute__((ext_vector_type(4)));
  extern __shared__ __align__(16) float tile_lds[];
  const int k_ld = dh + PT_PAD;                      // a key's row in LDS
  const int v_ld = WAVE + PT_PAD;                    // a dim's row of values in LDS
  const int p_ld = WAVE + PT_PAD;                    // a query's row of probabilities in LDS
  float* q_lds = tile_lds;                           // [PT_QUERIES][dh]
  float* k_lds = q_lds + PT_QUERIES * dh;            // [64][k_ld]
  float* v_lds = k_lds + WAVE * k_ld;                // [dh][v_ld]
  float* p_lds = v_lds + dh * v_ld;                  // [PA_WAVES][PT_PER_WAVE][p_ld]
  const int subtiles = tile_tokens / PT_QUERIES;
  const int tile = blockIdx.x / subtiles;
  const int head = blockIdx.y;
  const int run = blockIdx.z;
  const int lane_of_tile = query_tiles[2 * tile];
  if (lane_of_tile < 0) return;                      // a row of the table that holds nothing (a step of fixed capacity)
  const int first_row = query_tiles[2 * tile + 1] + (blockIdx.x - tile * subtiles) * PT_QUERIES;
  const int lane_end = cu_seqlens[lane_of_tile + 1];
  const int tile_end = min(query_tiles[2 * tile + 1] + tile_tokens, lane_end);
  const int count = min(PT_QUERIES, tile_end - first_row);          // queries of this workgroup
  if (count <= 0) return;
  const int last_position = positions[first_row + count - 1];      // positions ascend within a lane
  const int first_position = positions[first_row];
  int tile_first_key = 0;                                           // the oldest key any query of the tile sees
  if (window > 0 && first_position - window + 1 > 0) tile_first_key = first_position - window + 1;
  if (run * PA_RUN > last_position || (run + 1) * PA_RUN <= tile_first_key) return;
  const int kvh = head / (Hq / Hkv);
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int* table = block_tables + (long)lane_of_tile * max_pages;
  for (int index = tid; index < count * dh; index += PA_RUN) {
    const int query = index / dh;
    q_lds[index] = to_float(q[(long)(first_row + query) * q_ld + (long)head * dh + (index - query * dh)]);
  }
  // what a wave keeps of its queries' groups: (maximum, normalizer, sums of lane's dims), group by group
  float group_max[PT_PER_WAVE][PA_WAVES], group_norm[PT_PER_WAVE][PA_WAVES], group_o[PT_PER_WAVE][PA_WAVES][DIMS];
#pragma unroll
  for (int i = 0; i < PT_PER_WAVE; ++i)
#pragma unroll
    for (int g = 0; g < PA_WAVES; ++g) {
      group_max[i][g] = -INFINITY;
      group_norm[i][g] = 0.f;
#pragma unroll
      for (int d = 0; d < DIMS; ++d) group_o[i][g][d] = 0.f;
    }
  int query_position[PT_PER_WAVE];
#pragma unroll
  for (int i = 0; i < PT_PER_WAVE; ++i) {
    const int query = wave + i * PA_WAVES;
    query_position[i] = query < count ? positions[first_row + query] : -1;
  }

  // one group of 64 keys; called with a constant group so that what a wave keeps of it stays in registers
  auto take_group = [&](auto group_constant) {
    constexpr int g = decltype(group_constant)::value;
    const int group_first = run * PA_RUN + g * WAVE;
    if (group_first > last_position || group_first + WAVE <= tile_first_key) return;       // the same for every thread
    __syncthreads();                                    // the group before is read (and the queries are laid down)
    // keys group_first .. group_first + 63 that some query of the tile sees; the others (cells never written,
    // pages the request does not hold) are not fetched and lie in LDS as zeros that nobody multiplies
    const int keys = min(WAVE, last_position - group_first + 1);
    const int skipped = max(0, tile_first_key - group_first);      // keys before every query's window: their pages may be gone
    {
      // keys: four threads a key, each a quarter of its dims, 4 dims a load
      const int key_in = tid >> 2;
      const int quarter = dh >> 2;
      const int dim0 = (tid & 3) * quarter;
      float* to = k_lds + key_in * k_ld + dim0;
      if (key_in < keys && key_in >= skipped) {
        const int key = group_first + key_in;
        const int page = table[key / page_size];
        const T* from = k_base + (long)page * page_stride + ((long)kvh * page_size + key % page_size) * dh + dim0;
        for (int d = 0; d < quarter; d += 4) {
          const vec4 piece = *reinterpret_cast<const vec4*>(from + d);
          *reinterpret_cast<float4*>(to + d) = make_float4(to_float<T>(piece[0]), to_float<T>(piece[1]),
                                                           to_float<T>(piece[2]), to_float<T>(piece[3]));
        }
      } else {
        for (int d = 0; d < quarter; d += 4) *reinterpret_cast<float4*>(to + d) = make_float4(0.f, 0.f, 0.f, 0.f);
      }
    }
    {
      // values: a thread a key (the lanes of a wave walk along a page's tokens), the waves take every fourth dim
      const int key_in = lane;
      if (key_in < keys && key_in >= skipped) {
        const int key = group_first + key_in;
        const int page = table[key / page_size];
        const T* from = v_base + (long)page * page_stride + (long)kvh * dh * page_size + key % page_size;
        for (int dim = wave; dim < dh; dim += PA_WAVES) v_lds[dim * v_ld + key_in] = to_float(from[(long)dim * page_size]);
      } else {
        for (int dim = wave; dim < dh; dim += PA_WAVES) v_lds[dim * v_ld + key_in] = 0.f;
      }
    }
    __syncthreads();
    // the wave's four queries together: a key's dims and a key's values come out of LDS once for the four (LDS, not
    // the arithmetic, is what this kernel waits for); every query's products and sums are the ones of the per-token
    // kernel in their order.  A query that sees no key of the group ends with what its group started with
    // (maximum -inf, zeros); a query slot past the tile's last is computed on whatever LDS holds and never stored.
    float dot[PT_PER_WAVE];
#pragma unroll
    for (int i = 0; i < PT_PER_WAVE; ++i) dot[i] = 0.f;
    {
      const float* k_row = k_lds + lane * k_ld;
      for (int d = 0; d < dh; d += 4) {
        const float4 kv = *reinterpret_cast<const float4*>(k_row + d);
#pragma unroll
        for (int i = 0; i < PT_PER_WAVE; ++i) {
          const float4 qv = *reinterpret_cast<const float4*>(q_lds + (wave + i * PA_WAVES) * dh + d);
          dot[i] = fmaf(qv.x, kv.x, dot[i]);
          dot[i] = fmaf(qv.y, kv.y, dot[i]);
          dot[i] = fmaf(qv.z, kv.z, dot[i]);
          dot[i] = fmaf(qv.w, kv.w, dot[i]);
        }
      }
    }
    float* p_rows = p_lds + wave * (PT_PER_WAVE * p_ld);          // this wave's four rows of probabilities: no barrier, the wave runs in step
#pragma unroll
    for (int i = 0; i < PT_PER_WAVE; ++i) {
      const int position = query_position[i];
      int first_key = 0;
      if (window > 0 && position - window + 1 > 0) first_key = position - window + 1;
      const int key = group_first + lane;
      const bool visible = key >= first_key && key <= position;
      float score = -INFINITY;
      if (visible) {
        score = dot[i] * scale;
        if (slopes) score = fmaf(-slopes[head], (float)(position - key), score);
      }
      const float maximum = wave_max_dpp(score);
      const float p = visible ? (FAST_EXP ? __expf(score - maximum) : expf(score - maximum)) : 0.f;
      p_rows[i * p_ld + lane] = p;
      group_max[i][g] = maximum;
    }
    __builtin_amdgcn_wave_barrier();
    // sums over all 64 keys of the group: a key the query does not see has the probability 0 and a finite
    // value (a key some query of the tile sees, or a zero laid down above), so it adds an exact zero and the
    // sums are those of the keys from `from` to `to` in their order, which is what the per-token kernel adds
    {
      float sums[PT_PER_WAVE][DIMS];
#pragma unroll
      for (int i = 0; i < PT_PER_WAVE; ++i)
#pragma unroll
        for (int d = 0; d < DIMS; ++d) sums[i][d] = 0.f;
      const float* v_row[DIMS];
#pragma unroll
      for (int d = 0; d < DIMS; ++d) v_row[d] = v_lds + min(lane + d * WAVE, dh - 1) * v_ld;
      // the normalizers: lane i adds the probabilities of query i in the order of the keys
      const float* p_mine = p_rows + (lane & (PT_PER_WAVE - 1)) * p_ld;
      float normalizer = 0.f;
#pragma unroll
      for (int j = 0; j < WAVE; j += 4) {
        const float4 mine = *reinterpret_cast<const float4*>(p_mine + j);
        normalizer += mine.x;
        normalizer += mine.y;
        normalizer += mine.z;
        normalizer += mine.w;
        float4 pj[PT_PER_WAVE];
#pragma unroll
        for (int i = 0; i < PT_PER_WAVE; ++i) pj[i] = *reinterpret_cast<const float4*>(p_rows + i * p_ld + j);
#pragma unroll
        for (int d = 0; d < DIMS; ++d) {
          if (d * WAVE < dh) {                          // the same for every lane
            const float4 vj = *reinterpret_cast<const float4*>(v_row[d] + j);
#pragma unroll
            for (int i = 0; i < PT_PER_WAVE; ++i) {
              sums[i][d] = fmaf(pj[i].x, vj.x, sums[i][d]);
              sums[i][d] = fmaf(pj[i].y, vj.y, sums[i][d]);
              sums[i][d] = fmaf(pj[i].z, vj.z, sums[i][d]);
              sums[i][d] = fmaf(pj[i].w, vj.w, sums[i][d]);
            }
          }
        }
      }
#pragma unroll
      for (int i = 0; i < PT_PER_WAVE; ++i) {
        group_norm[i][g] = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, normalizer), i));
#pragma unroll
        for (int d = 0; d < DIMS; ++d) group_o[i][g][d] = sums[i][d];
      }
    }
    __builtin_amdgcn_wave_barrier();
  };
  take_group(std::integral_constant<int, 0>{});
  take_group(std::integral_constant<int, 1>{});
  take_group(std::integral_constant<int, 2>{});
  take_group(std::integral_constant<int, 3>{});
  static_assert(PA_WAVES == 4, "a run of keys is four groups of 64");
  // the groups of the run in their order, as the per-token kernel merges its waves
#pragma unroll
  for (int i = 0; i < PT_PER_WAVE; ++i) {
    const int position = query_position[i];
    int first_key = 0;
    if (window > 0 && position - window + 1 > 0) first_key = position - window + 1;
    if (position < 0 || (run + 1) * PA_RUN <= first_key || run * PA_RUN > position) continue;    // the per-token kernel writes nothing either
    float best = group_max[i][0];
#pragma unroll
    for (int g = 1; g < PA_WAVES; ++g) best = fmaxf(best, group_max[i][g]);
    float weight[PA_WAVES];
    float denominator = 0.f;
#pragma unroll
    for (int g = 0; g < PA_WAVES; ++g) {
      weight[g] = FAST_EXP ? __expf(group_max[i][g] - best) : expf(group_max[i][g] - best);
      denominator = fmaf(weight[g], group_norm[i][g], denominator);
    }
    const long token = first_row + wave + i * PA_WAVES;
    float* mine = partial + ((token * Hq + head) * runs + run) * (long)(dh + 2);
    if (lane == 0) {
      mine[0] = best;
      mine[1] = denominator;
    }
#pragma unroll
    for (int d = 0; d < DIMS; ++d) {
      const int dim = lane + d * WAVE;
      if (dim < dh) {
        float sum = 0.f;
#pragma unroll
        for (int g = 0; g < PA_WAVES; ++g) sum = fmaf(weight[g], group_o[i][g][d], sum);
        mine[2 + dim] = sum;
      }
    }
  }
}

template <typename T, bool FAST_EXP>
__global__ void paged_attention_merge_kernel(const float* __restrict__ partial, int Hq, int dh, int runs,
                                             const int* __restrict__ positions, int window,
                                             T* __restrict__ out, long out_ld) {
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int query_position = positions[token];
  int first_key = 0;
  if (window > 0 && query_position - window + 1 > 0) first_key = query_position - window + 1;
  const int first_run = first_key / PA_RUN;
  // a caller's bound on the contexts sizes the work area: a token beyond that bound merges the runs that
  // were launched for it and never reads outside the area
  const int last_run = min(query_position / PA_RUN, runs - 1);
  const float* theirs = partial + ((token * Hq + head) * runs) * (long)(dh + 2);
  for (int dim = threadIdx.x; dim < dh; dim += blockDim.x) {
    float maximum = -INFINITY, denominator = 0.f, sum = 0.f;
    for (int run = first_run; run <= last_run; ++run) {
      const float* one = theirs + (long)run * (dh + 2);
      const float larger = fmaxf(maximum, one[0]);
      const float keep = FAST_EXP ? __expf(maximum - larger) : expf(maximum - larger);     // 0 the first time
      const float weight = FAST_EXP ? __expf(one[0] - larger) : expf(one[0] - larger);
      denominator = denominator * keep + weight * one[1];
      sum = sum * keep + weight * one[2 + dim];
      maximum = larger;
    }
    out[token * out_ld + (long)head * dh + dim] = from_float<T>(sum / denominator);
  }
}

// partial: work area of at least T * Hq * runs * (dh + 2) floats, runs = ceil(max_seq_len / PA_RUN), where
// max_seq_len bounds the number of keys (position + 1) of every token of the step.
extern "C" long mi_paged_attention_workspace(int T, int Hq, int dh, int max_seq_len) {
  if (T <= 0 || Hq <= 0 || dh <= 0 || max_seq_len <= 0) return 0;
  return (long)T * Hq * ((max_seq_len + PA_RUN - 1) / PA_RUN) * (dh + 2);
}

// LDS of a workgroup of the tiled kernel: the tile's queries, 64 keys, their values, a wave's probabilities
static size_t paged_attention_tile_lds(int dh) {
  return ((size_t)PT_QUERIES * dh + (size_t)WAVE * (dh + PT_PAD) + (size_t)dh * (WAVE + PT_PAD) +
          (size_t)PT_QUERIES * (WAVE + PT_PAD)) * sizeof(float);
}

template <typename T, bool FAST_EXP, int DIMS>
static int raise_tile_lds(size_t bytes) {
  // beyond 64 KiB a kernel has to be told once per device that it may have that much (gfx950 has 160 KiB)
  static bool raised[64] = {};          // per instantiation of this function
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return ERR_BAD_ARGUMENT;
  if (raised[device]) return 0;
  if (hipFuncSetAttribute((const void*)paged_attention_tile_kernel<T, FAST_EXP, DIMS>, hipFuncAttributeMaxDynamicSharedMemorySize,
                          (int)bytes) != hipSuccess) {
    (void)hipGetLastError();
    return ERR_UNSUPPORTED_SIZE;
  }
  raised[device] = true;
  return 0;
}

// query_tiles (optional) [num_tiles, 2] = (lane or -1, first token row) of runs of up to tile_tokens tokens of one
// lane (tile_tokens a multiple of 16), with cu_seqlens [lanes + 1]: the step's lanes hold several tokens, and the
// partial results come from the kernel that shares a run's keys among the queries of a tile (the same bits).
extern "C" int mi_paged_attention(const void* q, int dtype, long q_ld, int T, int Hq, int Hkv, int dh,
                                  const void* k_base, const void* v_base, long page_stride, int page_size,
                                  const int* block_tables, int max_pages, const int* lane_of_token,
                                  const int* positions, float scale, int window, const float* slopes,
                                  int max_seq_len, float* partial, long partial_floats, void* out, long out_ld,
                                  const int* query_tiles, int num_tiles, int tile_tokens, const int* cu_seqlens,
                                  hipStream_t stream) {
  if (T <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || dh <= 0 || page_size <= 0 || max_pages <= 0 ||
      max_seq_len <= 0 || !partial)
    return ERR_BAD_ARGUMENT;
  if (dh > ATT_MAX_DH) return ERR_UNSUPPORTED_SIZE;
  const int runs = (max_seq_len + PA_RUN - 1) / PA_RUN;
  if (Hq > 65535 || runs > 65535) return ERR_UNSUPPORTED_SIZE;
  if (partial_floats < mi_paged_attention_workspace(T, Hq, dh, max_seq_len)) return ERR_BAD_ARGUMENT;
  const int element = dtype == DT_F32 ? 4 : 2;
  // the tiled kernel: head sizes in steps of 16, 4 elements a load from the cache
  bool tiled = query_tiles != nullptr && num_tiles > 0 && cu_seqlens != nullptr && tile_tokens > 0 &&
               tile_tokens % PT_QUERIES == 0 && dh % 16 == 0 && page_stride % 4 == 0 &&
               ((uintptr_t)k_base % (4 * element)) == 0 && (long)num_tiles * (tile_tokens / PT_QUERIES) <= 0x7fffffffL;
  const size_t tile_lds = paged_attention_tile_lds(dh);
  const int dims = dh <= WAVE ? 1 : dh <= 2 * WAVE ? 2 : 4;
  if (tiled && tile_lds > 64 * 1024) {
    int code;
    if (dtype == DT_F32) code = dims == 2 ? raise_tile_lds<float, false, 2>(tile_lds) : raise_tile_lds<float, false, 4>(tile_lds);
    else code = dims == 2 ? raise_tile_lds<bf16_t, true, 2>(tile_lds) : raise_tile_lds<bf16_t, true, 4>(tile_lds);
    if (code != 0) tiled = false;                      // the per-token kernel takes any size
  }
  const dim3 grid(T, Hq, runs);
  const dim3 tile_grid(tiled ? num_tiles * (tile_tokens / PT_QUERIES) : 1, Hq, runs);
  const dim3 merge_grid(T, Hq);
  const int merge_threads = dh <= WAVE ? WAVE : dh <= 2 * WAVE ? 2 * WAVE : 4 * WAVE;
  if (dtype == DT_F32) {
#define TILE_LAUNCH(T_, FAST_, DIMS_)                                                                                 \
  paged_attention_tile_kernel<T_, FAST_, DIMS_><<<tile_grid, PA_RUN, tile_lds, stream>>>(                              \
      (const T_*)q, q_ld, Hq, Hkv, dh, (const T_*)k_base, (const T_*)v_base, page_stride, page_size, block_tables,     \
      max_pages, query_tiles, tile_tokens, cu_seqlens, positions, scale, window, slopes, runs, partial)
    if (tiled && dims == 1) TILE_LAUNCH(float, false, 1);
    else if (tiled && dims == 2) TILE_LAUNCH(float, false, 2);
    else if (tiled) TILE_LAUNCH(float, false, 4);
    else
      paged_attention_kernel<float, false><<<grid, PA_RUN, 0, stream>>>(
          (const float*)q, q_ld, Hq, Hkv, dh, (const float*)k_base, (const float*)v_base, page_stride, page_size,
          block_tables, max_pages, lane_of_token, positions, scale, window, slopes, runs, partial);
    RETURN_IF_LAUNCH_FAILED();
    paged_attention_merge_kernel<float, false><<<merge_grid, merge_threads, 0, stream>>>(
        partial, Hq, dh, runs, positions, window, (float*)out, out_ld);
  } else if (dtype == DT_BF16) {
    if (tiled && dims == 1) TILE_LAUNCH(bf16_t, true, 1);
    else if (tiled && dims == 2) TILE_LAUNCH(bf16_t, true, 2);
    else if (tiled) TILE_LAUNCH(bf16_t, true, 4);
    else
      paged_attention_kernel<bf16_t, true><<<grid, PA_RUN, 0, stream>>>(
          (const bf16_t*)q, q_ld, Hq, Hkv, dh, (const bf16_t*)k_base, (const bf16_t*)v_base, page_stride,
          page_size, block_tables, max_pages, lane_of_token, positions, scale, window, slopes, runs, partial);
    RETURN_IF_LAUNCH_FAILED();
    paged_attention_merge_kernel<bf16_t, true><<<merge_grid, merge_threads, 0, stream>>>(
        partial, Hq, dh, runs, positions, window, (bf16_t*)out, out_ld);
  } else {
    return ERR_BAD_ARGUMENT;
  }
#undef TILE_LAUNCH
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- decode attention, split over the context
// For batches of single-token queries in bfloat16.  grid = (splits, kv heads, tokens); a block
// takes one page-aligned range of `split_keys` keys of one request and one kv head and serves
// all G query heads of that kv head from the same K and V loads:
//   scores : LPR = DH/8 lanes share a key row (16 B each), partial dots are summed across them;
//   softmax: over the block's range in float32 (scores staged in LDS), giving (max, sum);
//   values : V pages are [dim, token]; lane d owns output dim d and reads 8 tokens per load.
// Every block writes an unnormalized partial output with its (max, sum); the merge kernel
// combines the splits (the same (maximum, normalizer, accumulator) merge the reference does
// across simdgroups, crates/macllm-kernels/src/metal/paged_decode.metal:145-183).
#define DEC_THREADS 256
#define DEC_WAVES (DEC_THREADS / WAVE)
#define DEC_MAX_SPLIT 512

struct alignas(16) bf16x8 {
  bf16_t v[8];
};

template <int DH, int G>
__global__ void __launch_bounds__(DEC_THREADS)
decode_attention_kernel(const bf16_t* __restrict__ q, long q_ld, int Hq, const bf16_t* __restrict__ k_base,
                        const bf16_t* __restrict__ v_base, long page_stride, int page_size,
                        const int* __restrict__ block_tables, int max_pages,
                        const int* __restrict__ lane_of_token, const int* __restrict__ positions, float scale,
                        int window, int split_keys, int splits, float* __restrict__ partial_o,
                        float* __restrict__ partial_ml) {
  constexpr int LPR = DH / 8;
  constexpr int KPW = WAVE / LPR;
  constexpr int KPB = KPW * DEC_WAVES;
  constexpr int DPL = DH / WAVE;
  __shared__ float s_lds[G][DEC_MAX_SPLIT];
  __shared__ float red[DEC_WAVES][G];
  __shared__ float acc_lds[DEC_WAVES][G][DH];

  const int split = blockIdx.x;
  const int kvh = blockIdx.y;
  const long token = blockIdx.z;
  const int pos = positions[token];
  int first_key = 0;
  if (window > 0 && pos - window + 1 > 0) first_key = pos - window + 1;
  const int range_lo = (first_key / page_size) * page_size + split * split_keys;
  if (range_lo > pos) return;
  const int range_hi = min(range_lo + split_keys, pos + 1);
  const int count = range_hi - range_lo;
  const int* table = block_tables + (long)lane_of_token[token] * max_pages;
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int r = lane / LPR;
  const int c = lane % LPR;

  float qf[G][8];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    const bf16x8 packed = *reinterpret_cast<const bf16x8*>(q + token * q_ld + (long)(kvh * G + g) * DH + c * 8);
#pragma unroll
    for (int j = 0; j < 8; ++j) qf[g][j] = (float)packed.v[j] * scale;
  }

  // scores
  for (int base = 0; base < count; base += KPB) {
    const int local = base + wave * KPW + r;
    const int key = range_lo + local;
    const bool valid = local < count;
    float s[G];
#pragma unroll
    for (int g = 0; g < G; ++g) s[g] = 0.f;
    if (valid) {
      const int page = table[key / page_size];
      const int offset = key % page_size;
      const bf16x8 packed = *reinterpret_cast<const bf16x8*>(
          k_base + (long)page * page_stride + ((long)kvh * page_size + offset) * DH + c * 8);
      float kf[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) kf[j] = (float)packed.v[j];
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int j = 0; j < 8; ++j) s[g] = fmaf(qf[g][j], kf[j], s[g]);
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

  // softmax over the range: maximum, then exp and sum
  float m[G], l[G];
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = -INFINITY;
    for (int i = tid; i < count; i += DEC_THREADS) v = fmaxf(v, s_lds[g][i]);
    v = wave_max(v);
    if (lane == 0) red[wave][g] = v;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = red[0][g];
#pragma unroll
    for (int w = 1; w < DEC_WAVES; ++w) v = fmaxf(v, red[w][g]);
    m[g] = v;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float sum = 0.f;
    for (int i = tid; i < count; i += DEC_THREADS) {
      const float p = __expf(s_lds[g][i] - m[g]);
      s_lds[g][i] = p;
      sum += p;
    }
    sum = wave_sum(sum);
    if (lane == 0) red[wave][g] = sum;
  }
  __syncthreads();
#pragma unroll
  for (int g = 0; g < G; ++g) {
    float v = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) v += red[w][g];
    l[g] = v;
  }

  // values: each wave takes every fourth page of the range
  float acc[G][DPL];
#pragma unroll
  for (int g = 0; g < G; ++g)
#pragma unroll
    for (int i = 0; i < DPL; ++i) acc[g][i] = 0.f;
  const int range_pages = (count + page_size - 1) / page_size;
  for (int pg = wave; pg < range_pages; pg += DEC_WAVES) {
    const int local0 = pg * page_size;
    const int page = table[(range_lo + local0) / page_size];
    const int keys_here = min(page_size, count - local0);
#pragma unroll
    for (int i = 0; i < DPL; ++i) {
      const int dim = lane + i * WAVE;
      const bf16_t* v_row = v_base + (long)page * page_stride + ((long)kvh * DH + dim) * page_size;
      for (int j0 = 0; j0 < keys_here; j0 += 8) {
        const bf16x8 packed = *reinterpret_cast<const bf16x8*>(v_row + j0);
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          if (j0 + j < keys_here) {
            const float value = (float)packed.v[j];
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
    for (int i = 0; i < DPL; ++i) acc_lds[wave][g][lane + i * WAVE] = acc[g][i];
  __syncthreads();
  for (int index = tid; index < G * DH; index += DEC_THREADS) {
    const int g = index / DH;
    const int dim = index - g * DH;
    float sum = 0.f;
#pragma unroll
    for (int w = 0; w < DEC_WAVES; ++w) sum += acc_lds[w][g][dim];
    partial_o[((token * Hq + kvh * G + g) * splits + split) * DH + dim] = sum;
  }
  if (tid < G) {
    float* ml = partial_ml + ((token * Hq + kvh * G + tid) * splits + split) * 2;
    ml[0] = m[tid];
    ml[1] = l[tid];
  }
}

// out[token, head, :] = sum_s exp(m_s - M) o_s / sum_s exp(m_s - M) l_s over the splits that hold keys.
__global__ void decode_merge_kernel(const float* __restrict__ partial_o, const float* __restrict__ partial_ml,
                                    const int* __restrict__ positions, int window, int page_size,
                                    int split_keys, int splits, int Hq, int dh, bf16_t* __restrict__ out,
                                    long out_ld) {
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int pos = positions[token];
  int first_key = 0;
  if (window > 0 && pos - window + 1 > 0) first_key = pos - window + 1;
  const int first_page_key = (first_key / page_size) * page_size;
  const int used = min(splits, (pos - first_page_key) / split_keys + 1);
  const float* ml = partial_ml + (token * Hq + head) * splits * 2;
  const float* o = partial_o + (token * Hq + head) * (long)splits * dh;
  float maximum = -INFINITY;
  for (int s = 0; s < used; ++s) maximum = fmaxf(maximum, ml[2 * s]);
  float denominator = 0.f;
  for (int s = 0; s < used; ++s) denominator += __expf(ml[2 * s] - maximum) * ml[2 * s + 1];
  for (int dim = threadIdx.x; dim < dh; dim += blockDim.x) {
    float sum = 0.f;
    for (int s = 0; s < used; ++s) sum += __expf(ml[2 * s] - maximum) * o[(long)s * dh + dim];
    out[token * out_ld + (long)head * dh + dim] = (bf16_t)(sum / denominator);
  }
}

template <int DH, int G>
static int launch_decode(const bf16_t* q, long q_ld, int T, int Hq, int Hkv, const bf16_t* k_base,
                         const bf16_t* v_base, long page_stride, int page_size, const int* block_tables,
                         int max_pages, const int* lane_of_token, const int* positions, float scale, int window,
                         int split_keys, int splits, float* partial_o, float* partial_ml, hipStream_t stream) {
  const dim3 grid(splits, Hkv, T);
  decode_attention_kernel<DH, G><<<grid, DEC_THREADS, 0, stream>>>(
      q, q_ld, Hq, k_base, v_base, page_stride, page_size, block_tables, max_pages, lane_of_token, positions,
      scale, window, split_keys, splits, partial_o, partial_ml);
  return 0;
}

// Returns ERR_UNSUPPORTED_SIZE for shapes this kernel does not cover (the caller then uses
// mi_paged_attention): head_dim 64 or 128, 1..8 query heads per kv head, page_size a multiple of 8,
// split_keys a multiple of page_size and at most DEC_MAX_SPLIT.
extern "C" int mi_decode_attention(const void* q, long q_ld, int T, int Hq, int Hkv, int dh, const void* k_base,
                                   const void* v_base, long page_stride, int page_size, const int* block_tables,
                                   int max_pages, const int* lane_of_token, const int* positions, float scale,
                                   int window, int split_keys, int splits, float* partial_o, float* partial_ml,
                                   void* out, long out_ld, hipStream_t stream) {
  if (T <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || page_size <= 0 || splits <= 0 || max_pages <= 0)
    return ERR_BAD_ARGUMENT;
  const int G = Hq / Hkv;
  if ((dh != 64 && dh != 128) || G > 8 || page_size % 8 != 0 || split_keys % page_size != 0 ||
      split_keys <= 0 || split_keys > DEC_MAX_SPLIT || T > 65535 || Hkv > 65535)
    return ERR_UNSUPPORTED_SIZE;
#define DECODE_CASE(DH_, G_)                                                                                     \
  if (dh == DH_ && G == G_)                                                                                      \
    launch_decode<DH_, G_>((const bf16_t*)q, q_ld, T, Hq, Hkv, (const bf16_t*)k_base, (const bf16_t*)v_base,     \
                           page_stride, page_size, block_tables, max_pages, lane_of_token, positions, scale,     \
                           window, split_keys, splits, partial_o, partial_ml, stream);
  DECODE_CASE(64, 1) DECODE_CASE(64, 2) DECODE_CASE(64, 3) DECODE_CASE(64, 4) DECODE_CASE(64, 5)
  DECODE_CASE(64, 6) DECODE_CASE(64, 7) DECODE_CASE(64, 8)
  DECODE_CASE(128, 1) DECODE_CASE(128, 2) DECODE_CASE(128, 3) DECODE_CASE(128, 4) DECODE_CASE(128, 5)
  DECODE_CASE(128, 6) DECODE_CASE(128, 7) DECODE_CASE(128, 8)
#undef DECODE_CASE
  RETURN_IF_LAUNCH_FAILED();
  const dim3 merge_grid(T, Hq);
  decode_merge_kernel<<<merge_grid, dh, 0, stream>>>(partial_o, partial_ml, positions, window, page_size,
                                                     split_keys, splits, Hq, dh, (bf16_t*)out, out_ld);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- decode attention without a workspace argument
// The partial results live in an array of the library's device image (see static_scratch.h).  In host code
// the array's name is a stand-in, not a device address: its address on each GPU is asked for once per
// device, with that device current, and kept.
#include "static_scratch.h"
#include <mutex>

static __device__ __align__(256) float scratch[MI_STATIC_SCRATCH_BYTES / sizeof(float)];

#define STATIC_MAX_DEVICES 64
static float* scratch_of_device[STATIC_MAX_DEVICES];
static std::mutex scratch_lock;

// The address of this GPU's copy of `scratch`, or null with *error set.
static float* static_scratch(hipError_t* error) {
  int device = -1;
  *error = hipGetDevice(&device);
  if (*error != hipSuccess) return nullptr;
  if (device < 0 || device >= STATIC_MAX_DEVICES) {
    *error = hipErrorInvalidDevice;
    return nullptr;
  }
  std::lock_guard<std::mutex> guard(scratch_lock);
  if (scratch_of_device[device] == nullptr) {
    float* address = nullptr;
    *error = hipGetSymbolAddress((void**)&address, HIP_SYMBOL(scratch));
    if (*error != hipSuccess) return nullptr;
    scratch_of_device[device] = address;
  }
  return scratch_of_device[device];
}

extern "C" long mi_static_scratch_bytes(void) { return (long)MI_STATIC_SCRATCH_BYTES; }

extern "C" int mi_decode_attention_static(const void* q, long q_ld, int T, int Hq, int Hkv, int dh,
                                          const void* k_base, const void* v_base, long page_stride, int page_size,
                                          const int* block_tables, int max_pages, const int* lane_of_token,
                                          const int* positions, float scale, int window, int split_keys,
                                          int splits, void* out, long out_ld, hipStream_t stream) {
  if (T <= 0 || Hq <= 0 || dh <= 0 || splits <= 0) return ERR_BAD_ARGUMENT;
  // partial outputs first, their (max, sum) behind them, each part in whole runs of 256 bytes
  const unsigned long long rows = (unsigned long long)T * (unsigned long long)Hq * (unsigned long long)splits;
  const unsigned long long o_floats = (rows * (unsigned long long)dh + 63ull) & ~63ull;
  const unsigned long long ml_floats = (rows * 2ull + 63ull) & ~63ull;
  if (o_floats + ml_floats > MI_STATIC_SCRATCH_BYTES / sizeof(float)) return ERR_UNSUPPORTED_SIZE;
  hipError_t error = hipSuccess;
  float* base = static_scratch(&error);
  if (base == nullptr) return (int)error;
  return mi_decode_attention(q, q_ld, T, Hq, Hkv, dh, k_base, v_base, page_stride, page_size, block_tables,
                             max_pages, lane_of_token, positions, scale, window, split_keys, splits, base,
                             base + o_floats, out, out_ld, stream);
}

// ---------------------------------------------------------------- prefill attention on the matrix cores
// bfloat16, head_dim 64 or 128.  grid = (4 x query tiles, kv heads, head passes): a tile is up to 64
// consecutive tokens of one lane and a workgroup takes 16 of them with the query heads of one kv
// head (NSET column sets that share every K and V fragment).  The keys, from the first visible
// one to the workgroup's last position, are split in eight runs of whole 32-key steps, one per
// wave, read straight from the cache pages (the portion's own keys were written by rope_kv_store
// before), four steps in flight at a time; the eight partial results are merged through LDS,
// set by set.  Workgroups with the longest contexts (the last tiles) are launched first, in every
// other head pass last.
#include "attn_mfma.h"

#define PREFILL_STEPS 4
#define PREFILL_WAVES 8
#define PREFILL_FILL_BLOCKS 512   // two workgroups for each of the 256 compute units

template <int DH, int NSET>
__global__ void __launch_bounds__(PREFILL_WAVES * WAVE)
prefill_attention_kernel(const bf16_t* __restrict__ q, long q_ld, int Hq, int Hkv, const bf16_t* __restrict__ k_base,
                         const bf16_t* __restrict__ v_base, long page_stride, int page_size,
                         const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tiles,
                         const int* __restrict__ cu_seqlens, const int* __restrict__ start_pos, float scale,
                         int window, bf16_t* __restrict__ out, long out_ld) {
  constexpr int ITEMS = 2 + 4 * (DH / 16);                    // m, l and the accumulator of one set
  __shared__ float part[PREFILL_WAVES][ITEMS][WAVE];
  __shared__ int wave_pages[PREFILL_WAVES][WAVE];
  // heavy ones first; every other head pass the other way round, so that workgroups of two passes that
  // run side by side bring about the same work together
  const int block = (blockIdx.z & 1) ? blockIdx.x : gridDim.x - 1 - blockIdx.x;
  const int tile = block / 4;
  const int kvh = blockIdx.y;
  const int G = Hq / Hkv;
  const int head0 = kvh * G + blockIdx.z * NSET;             // first head of this pass
  const int request = tiles[2 * tile];
  if (request < 0) return;                                    // a row of the table past the step's own runs
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int qd = lane / 16;
  const int n = lane % 16;
  const int lane_end = cu_seqlens[request + 1];
  const int first_token = tiles[2 * tile + 1] + 16 * (block % 4);
  if (first_token >= lane_end) return;                        // the whole workgroup
  const int token = first_token + n;
  const bool has_query = token < lane_end;
  const int base_position = start_pos[request] - cu_seqlens[request];
  const int position = base_position + token;
  const int last_position = base_position + min(first_token + 15, lane_end - 1);
  const int first_position = base_position + first_token;
  // every column of the wave holds a query (16 tokens, and the head sets divide the heads): the wave's bounds are known
  const bool full_tile = first_token + 16 <= lane_end && (blockIdx.z + 1) * NSET <= G;

  mfma_bf16x8 q_frag[NSET][DH / 32];
  int col_pos[NSET];
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
    const bool valid = has_query && blockIdx.z * NSET + s < G;
    col_pos[s] = valid ? position : -1;
#pragma unroll
    for (int kk = 0; kk < DH / 32; ++kk) {
      if (valid) {
        q_frag[s][kk] = *reinterpret_cast<const mfma_bf16x8*>(q + (long)token * q_ld + (long)(head0 + s) * DH +
                                                               32 * kk + 8 * qd);
      } else {
#pragma unroll
        for (int j = 0; j < 8; ++j) q_frag[s][kk][j] = (bf16_t)0.f;
      }
    }
  }
  AttnAccumulator<DH, NSET> acc;
  acc.clear();
  AttnCache cache;
  cache.k_base = k_base;
  cache.v_base = v_base;
  cache.page_stride = page_stride;
  cache.page_size = page_size;
  cache.kvh = kvh;
  const int* cache_pages = block_tables + (long)request * max_pages;
  int key_lo = 0;
  if (window > 0 && first_position - window + 1 > 0) key_lo = ((first_position - window + 1) / 32) * 32;
  const int key_hi = last_position + 1;
  const int steps = (key_hi - key_lo + 31) / 32;
  const int steps_per_wave = (steps + PREFILL_WAVES - 1) / PREFILL_WAVES;
  const int my_lo = key_lo + 32 * steps_per_wave * wave;
  const int my_hi = min(key_hi, my_lo + 32 * steps_per_wave);
  // the page ids of the run go through LDS, 64 pages at a time (a wave's own corner of it: no
  // barrier), so that a K or V load does not wait for a load of its page id
  for (int part_lo = my_lo; part_lo < my_hi;) {
    const int first_page = part_lo / page_size;
    const int part_hi = min(my_hi, (first_page + WAVE) * page_size);
    wave_pages[wave][lane] = cache_pages[min(first_page + lane, max_pages - 1)];
    cache.pages = wave_pages[wave];
    cache.base_page = first_page;
    attend_keys<DH, NSET, PREFILL_STEPS>(acc, q_frag, col_pos, window, scale, part_lo, part_hi, cache,
                                         full_tile ? first_position : -1, last_position);
    part_lo = part_hi;
  }

  // merge: set s is finished by wave s
#pragma unroll
  for (int s = 0; s < NSET; ++s) {
    __syncthreads();
    part[wave][0][lane] = acc.m[s];
    part[wave][1][lane] = acc.l[s];
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt)
#pragma unroll
      for (int i = 0; i < 4; ++i) part[wave][2 + 4 * dt + i][lane] = acc.o[s][dt][i];
    __syncthreads();
    if (wave != s % PREFILL_WAVES) continue;
    float m = -INFINITY;
#pragma unroll
    for (int w = 0; w < PREFILL_WAVES; ++w) m = fmaxf(m, part[w][0][lane]);
    float factor[PREFILL_WAVES];
    float l = 0.f;
#pragma unroll
    for (int w = 0; w < PREFILL_WAVES; ++w) {
      const float m_w = part[w][0][lane];
      factor[w] = m_w == -INFINITY ? 0.f : __builtin_amdgcn_exp2f(m_w - m);
      l += part[w][1][lane] * factor[w];
    }
    l += __shfl_xor(l, 16, WAVE);
    l += __shfl_xor(l, 32, WAVE);
    if (col_pos[s] < 0) continue;
    const float inverse = 1.f / l;
    bf16_t* o = out + (long)token * out_ld + (long)(head0 + s) * DH;
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt) {
      mfma_bf16x4 packed;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float value = 0.f;
#pragma unroll
        for (int w = 0; w < PREFILL_WAVES; ++w) value += part[w][2 + 4 * dt + i][lane] * factor[w];
        packed[i] = (bf16_t)(value * inverse);
      }
      *reinterpret_cast<mfma_bf16x4*>(o + 16 * dt + 4 * qd) = packed;
    }
  }
}

// tiles: int32 [n_tiles, 2] = (lane, first token row of the tile); a tile never crosses a lane.
// Returns ERR_UNSUPPORTED_SIZE for shapes it does not cover (the caller uses mi_paged_attention).
extern "C" int mi_prefill_attention(const void* q, long q_ld, int Hq, int Hkv, int dh, const void* k_base,
                                    const void* v_base, long page_stride, int page_size, const int* block_tables,
                                    int max_pages, const int* tiles, int n_tiles, const int* cu_seqlens,
                                    const int* start_pos, float scale, int window, int max_seq_len, void* out,
                                    long out_ld, hipStream_t stream) {
  if (n_tiles <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || page_size <= 0 || max_pages <= 0)
    return ERR_BAD_ARGUMENT;
  const int G = Hq / Hkv;
  if ((dh != 64 && dh != 128) || page_size % 4 != 0 || q_ld % 8 != 0 || out_ld % 4 != 0 || Hkv > 65535 || G > 64)
    return ERR_UNSUPPORTED_SIZE;
  // up to four query heads share every K and V fragment; head size 128 holds twice the registers per head, and
  // more than two heads would spill.  A grid that would leave compute units with fewer than two workgroups, over
  // contexts of up to 2,048 keys (max_seq_len: an upper bound of the step's longest context, 0 = not known), is
  // bound by the softmax arithmetic of its longest tiles: it takes sets of two heads, so that twice the
  // workgroups, every other pass from the light end, spread that work.  Over longer contexts the keys and
  // values that four heads share count for more (a 2,048-token portion of the 0.5B shape behind 2,048 tokens
  // of context: 7.29 ms with two heads a set, 6.85 with four; behind 30,000 tokens 19.0 and 16.4).
  int most = dh == 128 ? 2 : 4;
  if (most > 2 && max_seq_len <= 2048 && 4L * n_tiles * Hkv * ((G + most - 1) / most) < PREFILL_FILL_BLOCKS) most = 2;
  const int passes = (G + most - 1) / most;
  const int nset = (G + passes - 1) / passes;
  if (n_tiles > (1 << 28)) return ERR_UNSUPPORTED_SIZE;
  const dim3 grid(4 * n_tiles, Hkv, passes);
#define PREFILL_CASE(DH_, NSET_)                                                                              \
  if (dh == DH_ && nset == NSET_)                                                                             \
    prefill_attention_kernel<DH_, NSET_><<<grid, PREFILL_WAVES * WAVE, 0, stream>>>(                                           \
        (const bf16_t*)q, q_ld, Hq, Hkv, (const bf16_t*)k_base, (const bf16_t*)v_base, page_stride, page_size, \
        block_tables, max_pages, tiles, cu_seqlens, start_pos, scale, window, (bf16_t*)out, out_ld);
  PREFILL_CASE(64, 1) PREFILL_CASE(64, 2) PREFILL_CASE(64, 3) PREFILL_CASE(64, 4)
  PREFILL_CASE(128, 1) PREFILL_CASE(128, 2) PREFILL_CASE(128, 3) PREFILL_CASE(128, 4)
#undef PREFILL_CASE
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
