// Sampling over rows of float32 logits [B, V]: penalties, greedy argmax, and
// temperature / top-k / top-p with one uniform draw per token.
//
// Order of operations (reference: src/sampling.rs:95-161):
//   repetition penalty over prompt+generated (x<0 ? x*p : x/p, :407-423), presence and
//   frequency penalties over generated tokens (:392-405), then either argmax with the
//   lowest index on ties (:425-433) or: divide by temperature, keep the k largest
//   (value descending, index ascending), softmax with the maximum subtracted, keep the
//   shortest descending prefix whose mass reaches top_p (:337-375), draw u * (kept mass)
//   and walk the kept tokens in index order (:165-169, :378-390).
// The uniform u comes from a counter-based generator: splitmix64 of
// seed + (draw_index + 1) * 0x9E3779B97F4A7C15, top 24 bits / 2^24.
#include "common.h"

#define SAMPLE_THREADS 1024

__device__ __forceinline__ unsigned int orderable(float v) {
  const unsigned int bits = __float_as_uint(v);
  return (bits & 0x80000000u) ? ~bits : (bits | 0x80000000u);   // ascending in v
}

__device__ __forceinline__ float from_orderable(unsigned int key) {
  const unsigned int bits = (key & 0x80000000u) ? (key & 0x7fffffffu) : ~key;
  return __uint_as_float(bits);
}

// ---------------------------------------------------------------- penalties
// tokens[offsets[b] .. offsets[b+1]) is row b's history (prompt then generated);
// the first prompt_lens[b] of them are the prompt.  count_all / count_gen are [B, V]
// int32 work areas that hold zeros on entry and on exit.  A row's newest generated token may still be
// on the device only: extra_rows[b] >= 0 names its place in extra_source, and it counts like the others.
__global__ void __launch_bounds__(SAMPLE_THREADS)
penalties_kernel(float* __restrict__ logits, int V, const int* __restrict__ tokens,
                 const int* __restrict__ offsets, const int* __restrict__ prompt_lens,
                 const float* __restrict__ repetition, const float* __restrict__ presence,
                 const float* __restrict__ frequency, int* __restrict__ count_all, int* __restrict__ count_gen,
                 const int* __restrict__ extra_source, const int* __restrict__ extra_rows) {
  const int row = blockIdx.x;
  float* values = logits + (long)row * V;
  int* all = count_all + (long)row * V;
  int* gen = count_gen + (long)row * V;
  const int begin = offsets[row];
  const int end = offsets[row + 1];
  const int prompt = prompt_lens[row];
  for (int i = begin + threadIdx.x; i < end; i += blockDim.x) {
    const int token = tokens[i];
    if (token < 0 || token >= V) continue;
    atomicAdd(&all[token], 1);
    if (i - begin >= prompt) atomicAdd(&gen[token], 1);
  }
  if (threadIdx.x == 0 && extra_source && extra_rows && extra_rows[row] >= 0) {
    const int token = extra_source[extra_rows[row]];
    if (token >= 0 && token < V) {
      atomicAdd(&all[token], 1);
      atomicAdd(&gen[token], 1);
    }
  }
  __threadfence();
  __syncthreads();
  const float rep = repetition[row];
  const bool use_rep = rep > 0.f && fabsf(rep - 1.0f) >= 1.1920929e-07f;
  const float pres = presence[row];
  const float freq = frequency[row];
  const bool use_openai = pres != 0.f || freq != 0.f;
  for (int v = threadIdx.x; v < V; v += blockDim.x) {
    const int seen = all[v];
    if (seen == 0) continue;
    float x = values[v];
    if (use_rep) x = x < 0.f ? x * rep : x / rep;
    const int generated = gen[v];
    if (use_openai && generated > 0) x -= freq * (float)generated + pres;
    values[v] = x;
    all[v] = 0;
    gen[v] = 0;
  }
}

extern "C" int mi_apply_penalties(float* logits, int B, int V, const int* tokens, const int* offsets,
                                  const int* prompt_lens, const float* repetition, const float* presence,
                                  const float* frequency, int* count_all, int* count_gen, const int* extra_source,
                                  const int* extra_rows, hipStream_t stream) {
  if (B <= 0 || V <= 0 || (extra_source == nullptr) != (extra_rows == nullptr)) return ERR_BAD_ARGUMENT;
  penalties_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, tokens, offsets, prompt_lens, repetition,
                                                     presence, frequency, count_all, count_gen, extra_source,
                                                     extra_rows);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- a constraint on the tokens
// Rows with a list of allowed tokens (ids[offsets[b] .. offsets[b + 1]), not empty) keep the logits of those and
// get -inf everywhere else; rows without one stay as they are.  After the penalties and before argmax or the draw
// (reference: src/sampling.rs:119-130, a constraint masks the penalized row).  One workgroup a row: the row's
// corner of `keep` (float32 [B, keep_ld]) is filled with -inf, takes the allowed logits, and is copied back.
__global__ void __launch_bounds__(SAMPLE_THREADS)
keep_allowed_kernel(float* __restrict__ logits, int V, const int* __restrict__ ids, const int* __restrict__ offsets,
                    float* __restrict__ keep, long keep_ld) {
  const int row = blockIdx.x;
  const int lo = offsets[row], hi = offsets[row + 1];
  if (lo >= hi) return;
  float* mine = logits + (long)row * V;
  float* kept = keep + (long)row * keep_ld;
  for (int v = threadIdx.x; v < V; v += blockDim.x) kept[v] = -INFINITY;
  __syncthreads();
  for (int j = lo + threadIdx.x; j < hi; j += blockDim.x) {
    const int id = ids[j];
    if (id >= 0 && id < V) kept[id] = mine[id];
  }
  __syncthreads();
  for (int v = threadIdx.x; v < V; v += blockDim.x) mine[v] = kept[v];
}

extern "C" int mi_keep_allowed(float* logits, int B, int V, const int* ids, const int* offsets, float* keep,
                               long keep_ld, hipStream_t stream) {
  if (B <= 0 || V <= 0 || !logits || !ids || !offsets || !keep || keep_ld < V) return ERR_BAD_ARGUMENT;
  keep_allowed_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, ids, offsets, keep, keep_ld);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- argmax
// (value descending, index ascending) packed so that the smallest 64-bit key wins.
__device__ __forceinline__ unsigned long long rank_key(float value, int index) {
  return ((unsigned long long)(~orderable(value)) << 32) | (unsigned int)index;
}

__device__ unsigned long long block_min_key(unsigned long long key, unsigned long long* scratch) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) {
    const unsigned long long other = __shfl_xor(key, offset, WAVE);
    key = other < key ? other : key;
  }
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  __syncthreads();
  if (lane == 0) scratch[wave] = key;
  __syncthreads();
  unsigned long long best = scratch[0];
  for (int i = 1; i < (int)(blockDim.x / WAVE); ++i) best = scratch[i] < best ? scratch[i] : best;
  return best;
}

// One workgroup a row.  The row is read in 16-byte pieces, eight of them asked for before the first is
// used (a row of 130,049 logits is 32 such pieces a thread); the elements before the first aligned piece
// and behind the last are read one by one (a row starts where the row before it ends, so at any alignment).
__global__ void __launch_bounds__(SAMPLE_THREADS)
argmax_kernel(const float* __restrict__ logits, int V, int* __restrict__ out) {
  __shared__ unsigned long long scratch[SAMPLE_THREADS / WAVE];
  typedef float float4_t __attribute__((ext_vector_type(4)));
  const float* values = logits + (long)blockIdx.x * V;
  const int head = min(V, (int)((4 - (((unsigned long long)values / sizeof(float)) & 3)) & 3));
  const int pieces = (V - head) / 4;
  unsigned long long best = ~0ull;
  auto take = [&](float value, int index) {
    const unsigned long long key = rank_key(value, index);
    best = key < best ? key : best;
  };
  if ((int)threadIdx.x < head) take(values[threadIdx.x], threadIdx.x);
  for (int v = head + 4 * pieces + threadIdx.x; v < V; v += blockDim.x) take(values[v], v);
  const float4_t* aligned = reinterpret_cast<const float4_t*>(values + head);
  constexpr int BATCH = 8;
  for (int first = threadIdx.x; first < pieces; first += BATCH * SAMPLE_THREADS) {
    float4_t piece[BATCH];
#pragma unroll
    for (int j = 0; j < BATCH; ++j) piece[j] = aligned[min(first + j * SAMPLE_THREADS, pieces - 1)];
#pragma unroll
    for (int j = 0; j < BATCH; ++j) {
      const int at = first + j * SAMPLE_THREADS;
      if (at < pieces) {
#pragma unroll
        for (int i = 0; i < 4; ++i) take(piece[j][i], head + 4 * at + i);
      }
    }
  }
  best = block_min_key(best, scratch);
  if (threadIdx.x == 0) out[blockIdx.x] = (int)(best & 0xffffffffu);
}

extern "C" int mi_argmax(const float* logits, int B, int V, int* out, hipStream_t stream) {
  if (B <= 0 || V <= 0) return ERR_BAD_ARGUMENT;
  argmax_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, out);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// ---------------------------------------------------------------- stochastic sampling
__device__ __forceinline__ float draw_uniform(unsigned long long seed, unsigned long long draw_index) {
  unsigned long long z = seed + (draw_index + 1ull) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  return (float)(z >> 40) * (1.0f / 16777216.0f);
}

// Exclusive prefix of per-thread sums over the block (thread order), plus the block total.
__device__ float block_exclusive_scan(float value, float* scratch /* blockDim.x floats */, float* total) {
  __syncthreads();
  scratch[threadIdx.x] = value;
  __syncthreads();
  // Hillis-Steele inclusive scan
  for (int offset = 1; offset < (int)blockDim.x; offset <<= 1) {
    float add = 0.f;
    if ((int)threadIdx.x >= offset) add = scratch[threadIdx.x - offset];
    __syncthreads();
    scratch[threadIdx.x] += add;
    __syncthreads();
  }
  const float inclusive = scratch[threadIdx.x];
  *total = scratch[blockDim.x - 1];
  return inclusive - value;
}

// One block per row.  `keys` is a [B, padded] 64-bit work area, padded = power of two >= V.
// Rows with temperature <= 0 take the argmax.  The row of logits is overwritten.
__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_kernel(float* __restrict__ logits, int V, int padded, const float* __restrict__ temperature,
              const int* __restrict__ top_k, const float* __restrict__ top_p,
              const unsigned long long* __restrict__ seeds, const int* __restrict__ draw_index,
              unsigned long long* __restrict__ keys, int* __restrict__ out, const int* __restrict__ done) {
  __shared__ float scan_scratch[SAMPLE_THREADS];
  __shared__ unsigned long long key_scratch[SAMPLE_THREADS / WAVE];
  __shared__ int found;
  const int row = blockIdx.x;
  if (done != nullptr && done[row] != 0) return;               // sample_select_kernel has drawn this row's token
  float* values = logits + (long)row * V;
  unsigned long long* sorted = keys + (long)row * padded;
  const float temp = temperature[row];

  if (temp <= 0.f) {
    unsigned long long best = ~0ull;
    for (int v = threadIdx.x; v < V; v += blockDim.x) {
      const unsigned long long key = rank_key(values[v], v);
      best = key < best ? key : best;
    }
    best = block_min_key(best, key_scratch);
    if (threadIdx.x == 0) out[row] = (int)(best & 0xffffffffu);
    return;
  }

  // scale and build sort keys
  for (int v = threadIdx.x; v < padded; v += blockDim.x) {
    if (v < V) {
      const float scaled = values[v] / temp;
      values[v] = scaled;
      sorted[v] = rank_key(scaled, v);
    } else {
      sorted[v] = ~0ull;
    }
  }
  __threadfence_block();
  __syncthreads();

  // bitonic sort, ascending keys = descending values, ties by ascending index
  for (int size = 2; size <= padded; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      for (int i = threadIdx.x; i < padded / 2; i += blockDim.x) {
        const int low = ((i / stride) * stride * 2) + (i % stride);
        const int high = low + stride;
        const bool ascending = ((low & size) == 0);
        const unsigned long long a = sorted[low];
        const unsigned long long b = sorted[high];
        if ((a > b) == ascending) {
          sorted[low] = b;
          sorted[high] = a;
        }
      }
      __threadfence_block();
      __syncthreads();
    }
  }

  int kept = V;
  const int k = top_k[row];
  if (k > 0 && k < V) kept = k;
  const float maximum = from_orderable(~(unsigned int)(sorted[0] >> 32));

  // softmax normalizer over the kept prefix
  const int chunk = (kept + blockDim.x - 1) / blockDim.x;
  const int chunk_begin = min(kept, (int)threadIdx.x * chunk);
  const int chunk_end = min(kept, chunk_begin + chunk);
  float local = 0.f;
  for (int i = chunk_begin; i < chunk_end; ++i)
    local += expf(from_orderable(~(unsigned int)(sorted[i] >> 32)) - maximum);
  float normalizer;
  float before = block_exclusive_scan(local, scan_scratch, &normalizer);

  // top-p: first sorted position whose cumulative probability reaches top_p
  const float p_limit = top_p[row];
  if (threadIdx.x == 0) found = kept;
  __syncthreads();
  if (p_limit >= 0.f && p_limit < 1.f) {
    // this thread's chunk starts at the scanned mass of its predecessors
    float cumulative = before / normalizer;
    for (int i = chunk_begin; i < chunk_end; ++i) {
      cumulative += expf(from_orderable(~(unsigned int)(sorted[i] >> 32)) - maximum) / normalizer;
      if (cumulative >= p_limit) {
        atomicMin(&found, i + 1);
        break;
      }
    }
  }
  __syncthreads();
  const int nucleus = found;
  __syncthreads();

  // probabilities of the kept tokens, scattered back in index order; zero elsewhere
  for (int v = threadIdx.x; v < V; v += blockDim.x) values[v] = 0.f;
  __threadfence_block();
  __syncthreads();
  for (int i = threadIdx.x; i < nucleus; i += blockDim.x) {
    const unsigned long long key = sorted[i];
    const int index = (int)(key & 0xffffffffu);
    values[index] = expf(from_orderable(~(unsigned int)(key >> 32)) - maximum) / normalizer;
  }
  __threadfence_block();
  __syncthreads();

  // walk in index order
  const int vchunk = (V + blockDim.x - 1) / blockDim.x;
  const int vbegin = min(V, (int)threadIdx.x * vchunk);
  const int vend = min(V, vbegin + vchunk);
  float mass = 0.f;
  for (int v = vbegin; v < vend; ++v) mass += values[v];
  float total;
  const float start = block_exclusive_scan(mass, scan_scratch, &total);
  const float target = draw_uniform(seeds[row], (unsigned long long)draw_index[row]) * total;
  if (threadIdx.x == 0) found = V;
  __syncthreads();
  float cumulative = start;
  for (int v = vbegin; v < vend; ++v) {
    const float p = values[v];
    if (p <= 0.f) continue;
    cumulative += p;
    if (target < cumulative) {
      atomicMin(&found, v);
      break;
    }
  }
  __syncthreads();
  if (threadIdx.x == 0) out[row] = found < V ? found : (int)(sorted[0] & 0xffffffffu);
}

// ---------------------------------------------------------------- the same without the full sort
// What is kept after top-k and top-p is small; sorting the whole vocabulary to find it is not
// needed.  With top-k (k <= SAMPLE_KMAX) the k smallest keys are found by a radix select over
// the 64-bit keys (eight passes of a 256-bin histogram), gathered and sorted in LDS; without
// top-k the SAMPLE_KMAX best candidates are taken the same way and the normalizer is summed over
// the whole row, and a nucleus that does not close within them (flat logits) gets its last token from a
// second radix select that counts mass instead of tokens; without top-k and top-p nothing is sorted at
// all.  The results are those of sample_kernel up to the rounding of float32 sums.  A row this kernel
// does not cover (k above SAMPLE_KMAX) is left with done[row] = 0 for sample_kernel, which skips the
// rows that are done.  The logits of a row that is drawn here are divided by its temperature in place.
#define SAMPLE_KMAX 1024
#define HISTOGRAM_COPIES 16
#define SAMPLE_LIST 2048             // keys that share their two upper bytes with the one looked for, listed in LDS
#define SAMPLE_ROW_PASSES_FROM 6     // the passes over bytes 7 and 6 read the row; those below read the list

// A row is read by one workgroup, which waits a microsecond for whatever it asks of memory: ROW_LOADS loads of a
// thread are asked for before the first is used (a row of 261,120 logits: 16 rounds instead of 255).
#define ROW_LOADS 16

// f(key) for every token of the row.  The row holds logits divided by the temperature; the first pass over it
// (SCALE) does the division and leaves the quotients in place: a division is a dozen instructions, and one
// workgroup's passes over a row are bound by its instructions.
template <bool SCALE, typename F>
__device__ __forceinline__ void for_each_key(float* __restrict__ values, int V, float temp, F f) {
  for (int base = threadIdx.x; base < V; base += ROW_LOADS * blockDim.x) {
    float x[ROW_LOADS];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) x[j] = values[min(base + j * (int)blockDim.x, V - 1)];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) {
      const int v = base + j * (int)blockDim.x;
      if (v < V) {
        if (SCALE) {
          x[j] = x[j] / temp;
          values[v] = x[j];
        }
        f(rank_key(x[j], v));
      }
    }
  }
}

// The sum of a value a thread over the block, added in a fixed order (lanes by halves, then the waves in turn).
__device__ float block_total(float value, float* scratch /* one float a wave */) {
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) value += __shfl_xor(value, offset, WAVE);
  __syncthreads();
  if ((threadIdx.x & (WAVE - 1)) == 0) scratch[threadIdx.x / WAVE] = value;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < (int)blockDim.x / WAVE; ++w) total += scratch[w];
  return total;
}

// The sum of f(value, v) over the row, consecutive lanes on consecutive tokens.
template <typename F>
__device__ float row_sum(const float* __restrict__ values, int V, float* scratch, F f) {
  float local = 0.f;
  for (int base = threadIdx.x; base < V; base += ROW_LOADS * blockDim.x) {
    float x[ROW_LOADS];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) x[j] = values[min(base + j * (int)blockDim.x, V - 1)];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) {
      const int v = base + j * (int)blockDim.x;
      if (v < V) local += f(x[j], v);
    }
  }
  return block_total(local, scratch);
}

// The first token, in index order, at which the running sum of mass(value, v) exceeds u times the sum
// over the row (V if there is none: rounding, when u is close to 1).  Every wave owns a run of consecutive
// tokens and sums it with consecutive lanes on consecutive tokens; the wave whose run holds the target then
// walks it 64 tokens at a time with a running sum across its lanes.
template <typename F>
__device__ int walk_in_index_order(const float* __restrict__ values, int V, float u, float* scratch, int* found,
                                   F mass) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int wave = threadIdx.x / WAVE;
  const int waves = blockDim.x / WAVE;
  const int run = ((V + waves - 1) / waves + WAVE - 1) / WAVE * WAVE;
  const int lo = min(V, wave * run);
  const int hi = min(V, lo + run);
  float local = 0.f;
  for (int base = lo + lane; base < hi; base += ROW_LOADS * WAVE) {
    float x[ROW_LOADS];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) x[j] = values[min(base + j * WAVE, V - 1)];
#pragma unroll
    for (int j = 0; j < ROW_LOADS; ++j) {
      const int v = base + j * WAVE;
      if (v < hi) local += mass(x[j], v);
    }
  }
#pragma unroll
  for (int offset = WAVE / 2; offset > 0; offset >>= 1) local += __shfl_xor(local, offset, WAVE);
  __syncthreads();
  if (lane == 0) scratch[wave] = local;
  if (threadIdx.x == 0) *found = V;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < waves; ++w) total += scratch[w];
  const float target = u * total;
  float before = 0.f;
  int holder = -1;
  for (int w = 0; w < waves; ++w) {
    if (holder < 0 && target < before + scratch[w]) holder = w;
    if (holder < 0) before += scratch[w];
  }
  if (wave == holder) {
    float running = before;
    for (int base = lo; base < hi; base += WAVE) {
      const int v = base + lane;
      const float p = v < hi ? mass(values[min(v, V - 1)], v) : 0.f;
      float inclusive = p;
#pragma unroll
      for (int offset = 1; offset < WAVE; offset <<= 1) {
        const float other = __shfl_up(inclusive, offset, WAVE);
        if (lane >= offset) inclusive += other;
      }
      const unsigned long long crossed = __ballot(p > 0.f && target < running + inclusive);
      if (crossed != 0ull) {
        if (lane == 0) *found = base + __ffsll((long long)crossed) - 1;
        break;
      }
      running += __shfl(inclusive, WAVE - 1, WAVE);
    }
  }
  __syncthreads();
  return *found;
}

__device__ void lds_bitonic_sort(unsigned long long* keys, int padded) {
  for (int size = 2; size <= padded; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      __syncthreads();
      for (int i = threadIdx.x; i < padded / 2; i += blockDim.x) {
        const int low = ((i / stride) * stride * 2) + (i % stride);
        const int high = low + stride;
        const bool ascending = ((low & size) == 0);
        const unsigned long long a = keys[low];
        const unsigned long long b = keys[high];
        if ((a > b) == ascending) {
          keys[low] = b;
          keys[high] = a;
        }
      }
    }
  }
  __syncthreads();
}

__global__ void __launch_bounds__(SAMPLE_THREADS)
sample_select_kernel(float* __restrict__ logits, int V, const float* __restrict__ temperature,
                     const int* __restrict__ top_k, const float* __restrict__ top_p,
                     const unsigned long long* __restrict__ seeds, const int* __restrict__ draw_index,
                     int* __restrict__ out, int* __restrict__ done) {
  __shared__ float scan_scratch[SAMPLE_THREADS];
  __shared__ unsigned long long key_scratch[SAMPLE_THREADS / WAVE];
  __shared__ unsigned long long candidates[SAMPLE_KMAX];
  __shared__ unsigned long long by_index[SAMPLE_KMAX];
  __shared__ unsigned int histogram[256];
  __shared__ unsigned int histogram_copies[HISTOGRAM_COPIES][256];   // the passes over the row count into the copy of their lane
  __shared__ unsigned long long mass_histogram[256];
  __shared__ unsigned long long chosen_prefix, remaining_mass;
  __shared__ unsigned long long list[SAMPLE_LIST];
  __shared__ int listed;
  __shared__ int remaining, found, gathered, bin_taken_whole;
  const int row = blockIdx.x;
  const int tid = threadIdx.x;
  float* values = logits + (long)row * V;          // divided by the temperature in the first pass over them
  const float temp = temperature[row];
  if (tid == 0) done[row] = 0;

  if (temp <= 0.f) {
    unsigned long long best = ~0ull;
    for (int v = tid; v < V; v += blockDim.x) {
      const unsigned long long key = rank_key(values[v], v);
      best = key < best ? key : best;
    }
    best = block_min_key(best, key_scratch);
    if (tid == 0) {
      out[row] = (int)(best & 0xffffffffu);
      done[row] = 1;
    }
    return;
  }
  const int k = top_k[row];
  const bool use_top_k = k > 0 && k < V;
  const float p_limit = top_p[row];
  const bool use_top_p = p_limit >= 0.f && p_limit < 1.f;
  if (use_top_k && k > SAMPLE_KMAX) return;                    // sample_kernel's
  const float u = draw_uniform(seeds[row], (unsigned long long)draw_index[row]);

  if (!use_top_k && !use_top_p) {
    // every token is kept: maximum, normalizer, and the walk in index order
    unsigned long long best = ~0ull;
    for_each_key<true>(values, V, temp, [&](unsigned long long key) { best = key < best ? key : best; });
    best = block_min_key(best, key_scratch);
    const float maximum = from_orderable(~(unsigned int)(best >> 32));
    const float normalizer = row_sum(values, V, scan_scratch, [&](float scaled, int) { return expf(scaled - maximum); });
    const int token = walk_in_index_order(values, V, u, scan_scratch, &found,
                                          [&](float scaled, int) { return expf(scaled - maximum) / normalizer; });
    if (tid == 0) {
      out[row] = token < V ? token : (int)(best & 0xffffffffu);
      done[row] = 1;
    }
    return;
  }

  // ---- the K smallest keys: radix select of the K-th, most significant byte first
  const int K = use_top_k ? k : min(V, SAMPLE_KMAX);
  if (tid == 0) {
    chosen_prefix = 0ull;
    remaining = K;
  }
  if (tid == 0) listed = 0;
  for (int pass = 7; pass >= 0; --pass) {
    if (tid < 256) histogram[tid] = 0u;
    for (int i = tid; i < HISTOGRAM_COPIES * 256; i += blockDim.x) (&histogram_copies[0][0])[i] = 0u;
    __syncthreads();
    const unsigned long long prefix = chosen_prefix;
    const unsigned long long above = pass == 7 ? 0ull : (~0ull << (8 * (pass + 1)));
    if (pass == SAMPLE_ROW_PASSES_FROM - 1) {
      // two bytes of the keys are fixed: the keys that still match are few; they are listed, and the bytes below
      // are found among them instead of in passes over the row (when they fit the list)
      for_each_key<false>(values, V, temp, [&](unsigned long long key) {
        if ((key & above) == prefix) {
          const int slot = atomicAdd(&listed, 1);
          if (slot < SAMPLE_LIST) list[slot] = key;
        }
      });
      __syncthreads();
    }
    auto count = [&](unsigned long long key) {
      if ((key & above) == prefix) atomicAdd(&histogram[(unsigned int)(key >> (8 * pass)) & 255u], 1u);
    };
    // over the row, nearly all keys of the top bytes fall into a few bins, and additions of one wave to one LDS
    // address are done one after the other: every lane counts into one of HISTOGRAM_COPIES copies, added up after
    auto count_row = [&](unsigned long long key) {
      if ((key & above) == prefix)
        atomicAdd(&histogram_copies[tid % HISTOGRAM_COPIES][(unsigned int)(key >> (8 * pass)) & 255u], 1u);
    };
    bool over_the_row = true;
    if (pass < SAMPLE_ROW_PASSES_FROM && listed <= SAMPLE_LIST) {
      for (int i = tid; i < listed; i += blockDim.x) count(list[i]);
      over_the_row = false;
    } else if (pass == 7) {
      for_each_key<true>(values, V, temp, count_row);
    } else {
      for_each_key<false>(values, V, temp, count_row);
    }
    __syncthreads();
    if (over_the_row && tid < 256) {
      unsigned int sum = 0u;
#pragma unroll
      for (int copy = 0; copy < HISTOGRAM_COPIES; ++copy) sum += histogram_copies[copy][tid];
      histogram[tid] = sum;
    }
    __syncthreads();
    // the bin in which the running count reaches what is still wanted: the first wave scans the
    // 256 bins, four a lane
    if (tid < WAVE) {
      const int left = remaining;
      unsigned int mine[4], sum = 0u;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mine[j] = histogram[4 * tid + j];
        sum += mine[j];
      }
      unsigned int inclusive = sum;
#pragma unroll
      for (int offset = 1; offset < WAVE; offset <<= 1) {
        const unsigned int other = __shfl_up(inclusive, offset, WAVE);
        if (tid >= offset) inclusive += other;
      }
      unsigned int before = inclusive - sum;
      if ((int)before < left && (int)inclusive >= left) {          // exactly one lane
        int bin = 4 * tid;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
          if ((int)(before + mine[j]) < left) {
            before += mine[j];
            ++bin;
          } else {
            break;
          }
        }
        remaining = left - (int)before;
        chosen_prefix = prefix | ((unsigned long long)bin << (8 * pass));
        // every key of the bin is wanted: the K-th is the bin's largest, whatever its lower bytes
        bin_taken_whole = (int)histogram[bin] == left - (int)before ? 1 : 0;
      }
    }
    __syncthreads();
    if (bin_taken_whole) {
      if (tid == 0 && pass > 0) chosen_prefix |= (~0ull >> (64 - 8 * pass));
      __syncthreads();
      break;
    }
  }
  const unsigned long long kth = chosen_prefix;
  int padded = 1;
  while (padded < K) padded <<= 1;
  for (int i = tid; i < padded; i += blockDim.x) candidates[i] = ~0ull;
  if (tid == 0) gathered = 0;
  __syncthreads();
  for_each_key<false>(values, V, temp, [&](unsigned long long key) {
    if (key <= kth) {
      const int slot = atomicAdd(&gathered, 1);
      if (slot < SAMPLE_KMAX) candidates[slot] = key;
    }
  });
  lds_bitonic_sort(candidates, padded);                        // descending values, ties by ascending index
  const float maximum = from_orderable(~(unsigned int)(candidates[0] >> 32));

  // ---- softmax normalizer: over the kept tokens (top-k), or over the whole row
  float normalizer;
  const int chunk = (K + blockDim.x - 1) / blockDim.x;
  const int chunk_begin = min(K, tid * chunk);
  const int chunk_end = min(K, chunk_begin + chunk);
  float local = 0.f;
  for (int i = chunk_begin; i < chunk_end; ++i)
    local += expf(from_orderable(~(unsigned int)(candidates[i] >> 32)) - maximum);
  float candidate_mass;
  const float before = block_exclusive_scan(local, scan_scratch, &candidate_mass);
  if (use_top_k) {
    normalizer = candidate_mass;
  } else {
    normalizer = row_sum(values, V, scan_scratch, [&](float scaled, int) { return expf(scaled - maximum); });
  }

  // ---- top-p: the shortest prefix in sorted order whose mass reaches top_p
  constexpr int OPEN = 0x7fffffff;
  if (tid == 0) found = OPEN;
  __syncthreads();
  if (use_top_p) {
    float cumulative = before / normalizer;
    for (int i = chunk_begin; i < chunk_end; ++i) {
      cumulative += expf(from_orderable(~(unsigned int)(candidates[i] >> 32)) - maximum) / normalizer;
      if (cumulative >= p_limit) {
        atomicMin(&found, i + 1);
        break;
      }
    }
  }
  __syncthreads();
  const int closed_at = found;
  __syncthreads();
  if (closed_at == OPEN && !use_top_k && K < V) {
    // ---- the nucleus is wider than the candidates (flat logits): its last token by a radix select over the
    // keys again, this time counting mass instead of tokens.  Masses are fixed-point (probability * 2^40,
    // 64-bit sums: exact, so every pass sees the same totals whatever the order of the additions): the bin in
    // which the running mass reaches what is still wanted is taken, byte by byte, down to one key.
    const float fixed_one = 1099511627776.f;
    if (tid == 0) {
      chosen_prefix = 0ull;
      remaining_mass = (unsigned long long)(p_limit * fixed_one);
    }
    for (int pass = 7; pass >= 0; --pass) {
      if (tid < 256) mass_histogram[tid] = 0ull;
      __syncthreads();
      const unsigned long long prefix = chosen_prefix;
      const unsigned long long above = pass == 7 ? 0ull : (~0ull << (8 * (pass + 1)));
      auto add_mass = [&](unsigned long long key) {
        if ((key & above) == prefix)
          atomicAdd(&mass_histogram[(unsigned int)(key >> (8 * pass)) & 255u],
                    (unsigned long long)(expf(from_orderable(~(unsigned int)(key >> 32)) - maximum) / normalizer * fixed_one));
      };
      if (pass == SAMPLE_ROW_PASSES_FROM - 1) {
        if (tid == 0) listed = 0;
        __syncthreads();
        for_each_key<false>(values, V, temp, [&](unsigned long long key) {
          if ((key & above) == prefix) {
            const int slot = atomicAdd(&listed, 1);
            if (slot < SAMPLE_LIST) list[slot] = key;
          }
        });
        __syncthreads();
      }
      if (pass < SAMPLE_ROW_PASSES_FROM && listed <= SAMPLE_LIST) {
        for (int i = tid; i < listed; i += blockDim.x) add_mass(list[i]);
      } else {
        for_each_key<false>(values, V, temp, add_mass);
      }
      __syncthreads();
      if (tid < WAVE) {
        unsigned long long mine[4], sum = 0ull;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          mine[j] = mass_histogram[4 * tid + j];
          sum += mine[j];
        }
        unsigned long long inclusive = sum;
#pragma unroll
        for (int offset = 1; offset < WAVE; offset <<= 1) {
          const unsigned long long other = __shfl_up(inclusive, offset, WAVE);
          if (tid >= offset) inclusive += other;
        }
        const unsigned long long all = __shfl(inclusive, WAVE - 1, WAVE);
        // what is wanted is at most what there is (the top pass; below it the bin taken holds it by construction)
        const unsigned long long wanted = remaining_mass < all ? remaining_mass : all;
        unsigned long long before = inclusive - sum;
        if (sum > 0ull && before < wanted && inclusive >= wanted) {      // exactly one lane (none if wanted is 0)
          int bin = 4 * tid;
#pragma unroll
          for (int j = 0; j < 3; ++j) {
            if (before + mine[j] < wanted) {
              before += mine[j];
              ++bin;
            } else {
              break;
            }
          }
          remaining_mass = wanted - before;
          chosen_prefix = prefix | ((unsigned long long)bin << (8 * pass));
        }
      }
      __syncthreads();
    }
    const unsigned long long last_kept = remaining_mass > 0ull ? chosen_prefix : candidates[0];
    // ---- walk the kept tokens in index order
    const int token = walk_in_index_order(values, V, u, scan_scratch, &found, [&](float scaled, int v) {
      return rank_key(scaled, v) <= last_kept ? expf(scaled - maximum) / normalizer : 0.f;
    });
    if (tid == 0) {
      out[row] = token < V ? token : (int)(candidates[0] & 0xffffffffu);
      done[row] = 1;
    }
    return;
  }
  const int nucleus = min(closed_at, K);

  // ---- walk the nucleus in index order
  int padded_nucleus = 1;
  while (padded_nucleus < nucleus) padded_nucleus <<= 1;
  for (int i = tid; i < padded_nucleus; i += blockDim.x)
    by_index[i] = i < nucleus ? ((candidates[i] & 0xffffffffull) << 32) | (unsigned long long)i : ~0ull;
  lds_bitonic_sort(by_index, padded_nucleus);
  const int nchunk = (nucleus + blockDim.x - 1) / blockDim.x;
  const int nbegin = min(nucleus, tid * nchunk);
  const int nend = min(nucleus, nbegin + nchunk);
  auto probability = [&](int position) {
    const unsigned long long key = candidates[(int)(by_index[position] & 0xffffffffull)];
    return expf(from_orderable(~(unsigned int)(key >> 32)) - maximum) / normalizer;
  };
  float mass = 0.f;
  for (int i = nbegin; i < nend; ++i) mass += probability(i);
  float total;
  const float start = block_exclusive_scan(mass, scan_scratch, &total);
  const float target = u * total;
  if (tid == 0) found = nucleus;
  __syncthreads();
  float cumulative = start;
  for (int i = nbegin; i < nend; ++i) {
    const float p = probability(i);
    if (p <= 0.f) continue;
    cumulative += p;
    if (target < cumulative) {
      atomicMin(&found, i);
      break;
    }
  }
  __syncthreads();
  if (tid == 0) {
    out[row] = found < nucleus ? (int)(by_index[found] >> 32) : (int)(candidates[0] & 0xffffffffu);
    done[row] = 1;
  }
}

extern "C" int mi_sample(float* logits, int B, int V, int padded, const float* temperature, const int* top_k,
                         const float* top_p, const unsigned long long* seeds, const int* draw_index,
                         unsigned long long* keys, int* out, int* done, hipStream_t stream) {
  if (B <= 0 || V <= 0 || padded < V || (padded & (padded - 1)) != 0) return ERR_BAD_ARGUMENT;
  // done: int32 [B] work area, or null to sort every row (the reference path of the tests)
  if (done != nullptr) {
    sample_select_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, temperature, top_k, top_p, seeds, draw_index,
                                                           out, done);
    RETURN_IF_LAUNCH_FAILED();
  }
  sample_kernel<<<B, SAMPLE_THREADS, 0, stream>>>(logits, V, padded, temperature, top_k, top_p, seeds,
                                                  draw_index, keys, out, done);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
