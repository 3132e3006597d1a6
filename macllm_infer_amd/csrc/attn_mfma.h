// Attention over the paged cache on the matrix cores (bfloat16, v_mfma_f32_16x16x32_bf16),
// one wavefront at a time, shared by the prefill kernel (columns = 16 queries of one head)
// and the decode kernel (columns = the query heads of one kv head).
//
// A wave works on NSET sets of 16 columns that read the same kv head, and walks a run of keys
// 32 at a time:
//   scores   S^T[key, col] = K[key, :] . Q[col, :]     A = K (16 keys x 32 dims, contiguous in
//            dims), B = Q^T (contiguous in dims): no transposes; the result lands with lane
//            (q, n) holding keys 4q..4q+3 of each 16-key tile for column n;
//   softmax  online, per column, in float32 (scores kept in units of log2 so that the
//            exponentials are bare exp2): running maximum and normalizer, the accumulator
//            rescaled when the maximum moves;
//   values   O^T[dim, col] += V^T[dim, key] . P^T[key, col]: V pages are stored [dim, token], so
//            A = V^T is contiguous in tokens, and the probabilities a lane holds after the
//            softmax (4 keys of tile 0, 4 keys of tile 1) are exactly its B fragment once the
//            32 keys of the step are numbered (q, j) -> j < 4 ? 4q + j : 16 + 4q + (j - 4).
// Formulas: s = q.k * scale, key visible when key <= column position and, with a window w,
// position - key < w (reference: src/decoder.rs:4515-4532, 4641-4670); softmax in float32.
#pragma once
#include "common.h"

typedef __bf16 mfma_bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 mfma_bf16x4 __attribute__((ext_vector_type(4)));
typedef float mfma_floatx4 __attribute__((ext_vector_type(4)));
typedef unsigned mfma_uintx4 __attribute__((ext_vector_type(4)));

template <int DH, int NSET>
struct AttnAccumulator {
  float m[NSET];                       // running maximum of this lane's column in each set, in units of log2 (merge with exp2)
  float l[NSET];                       // this lane's share of the normalizer (summed over q at the end)
  mfma_floatx4 o[NSET][DH / 16];       // O^T[dims 16*dt + 4q + i][column n]

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int s = 0; s < NSET; ++s) {
      m[s] = -INFINITY;
      l[s] = 0.f;
#pragma unroll
      for (int dt = 0; dt < DH / 16; ++dt) o[s][dt] = mfma_floatx4{0.f, 0.f, 0.f, 0.f};
    }
  }
};

struct AttnCache {
  const bf16_t* k_base;
  const bf16_t* v_base;
  long page_stride;
  int page_size;
  int kvh;
  const int* pages;      // page id of logical page (index + base_page); LDS or global
  int base_page;
};

// The K and V fragments of STEPS steps of 32 keys from key k00 on.  K: rows of two 16-key tiles
// per step; V^T: columns of the same 32 keys.  Keys past last_key are clamped to it (their cells
// are masked or zeroed by attn_compute).
template <int DH, int STEPS>
struct AttnFragments {
  mfma_bf16x8 k[STEPS][2][DH / 32];
  mfma_bf16x8 v[STEPS][DH / 16];
};

template <int DH, int STEPS>
__device__ __forceinline__ void attn_load(AttnFragments<DH, STEPS>& f, int k00, int last_key, const AttnCache& cache) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int q = lane / 16;
  const int r = lane % 16;
#pragma unroll
  for (int st = 0; st < STEPS; ++st) {
    const int k0 = k00 + 32 * st;
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(k0 + 16 * t + r, last_key);
      const int page = cache.pages[key / cache.page_size - cache.base_page];
      const bf16_t* row = cache.k_base + (long)page * cache.page_stride +
                          ((long)cache.kvh * cache.page_size + key % cache.page_size) * DH + 8 * q;
#pragma unroll
      for (int kk = 0; kk < DH / 32; ++kk) f.k[st][t][kk] = *reinterpret_cast<const mfma_bf16x8*>(row + 32 * kk);
    }
    int page[2], offset[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      const int key = min(k0 + 16 * t + 4 * q, last_key & ~3);
      page[t] = cache.pages[key / cache.page_size - cache.base_page];
      offset[t] = key % cache.page_size;
    }
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const mfma_bf16x4 part = *reinterpret_cast<const mfma_bf16x4*>(
            cache.v_base + (long)page[t] * cache.page_stride +
            ((long)cache.kvh * DH + 16 * dt + r) * cache.page_size + offset[t]);
#pragma unroll
        for (int j = 0; j < 4; ++j) f.v[st][dt][4 * t + j] = part[j];
      }
    }
  }
}

// Scores, softmax step and values of the loaded steps, per set of columns.
// MASKED = false: the caller vouches that every key of the round is visible to every column
// and lies inside the run (steps away from the diagonal, the window's edge and the run's end):
// no masks are computed.
template <int DH, int NSET, int STEPS, bool MASKED = true>
__device__ __forceinline__ void attn_compute(AttnAccumulator<DH, NSET>& acc, AttnFragments<DH, STEPS>& f,
                                             const mfma_bf16x8 (&q_frag)[NSET][DH / 32],
                                             const int (&col_pos)[NSET], int window, float scale, int k00,
                                             int key_hi) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int q = lane / 16;
  const int last_key = key_hi - 1;
  const float scale_log2 = scale * 1.4426950408889634f;
#pragma unroll
  for (int st = 0; st < STEPS; ++st) {
    const int k0 = k00 + 32 * st;
    if (k0 >= key_hi) break;
    // cells past the end of the run were never written: keep them out of the product (with bit
    // masks and without a branch, so that no wait for loads that are still under way is forced)
    if (MASKED) {
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        const int valid = last_key - (k0 + 16 * t + 4 * q) + 1;            // cells of this lane's four that hold keys
        const unsigned lo = valid >= 2 ? 0xffffffffu : (valid == 1 ? 0x0000ffffu : 0u);
        const unsigned hi = valid >= 4 ? 0xffffffffu : (valid == 3 ? 0x0000ffffu : 0u);
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) {
          mfma_uintx4 bits = __builtin_bit_cast(mfma_uintx4, f.v[st][dt]);
          bits[2 * t] &= lo;
          bits[2 * t + 1] &= hi;
          f.v[st][dt] = __builtin_bit_cast(mfma_bf16x8, bits);
        }
      }
    }
#pragma unroll
    for (int s = 0; s < NSET; ++s) {
      mfma_floatx4 score[2];
#pragma unroll
      for (int t = 0; t < 2; ++t) {
        score[t] = mfma_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int kk = 0; kk < DH / 32; ++kk)
          score[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.k[st][t][kk], q_frag[s][kk], score[t], 0, 0, 0);
      }
      // scores in units of log2: s * scale * log2(e), so that the exponentials are bare v_exp
      if (MASKED) {
        // visible keys of the column: first_visible .. min(position, last_key); relative to the step
        // they are lo .. lo + span, so one unsigned compare per score decides (an empty range gets
        // a lo that no offset reaches)
        const int position = col_pos[s];
        const int first_visible = window > 0 ? max(position - window + 1, 0) : 0;
        const int last_visible = min(position, last_key);
        const bool any = last_visible >= first_visible;
        const int lo = any ? first_visible - k0 : 0x40000000;
        const unsigned span = any ? (unsigned)(last_visible - first_visible) : 0u;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const bool visible = (unsigned)(16 * t + 4 * q + i - lo) <= span;
            score[t][i] = visible ? score[t][i] : -INFINITY;
          }
      }
      float step_max = fmaxf(fmaxf(fmaxf(score[0][0], score[0][1]), fmaxf(score[0][2], score[0][3])),
                             fmaxf(fmaxf(score[1][0], score[1][1]), fmaxf(score[1][2], score[1][3])));
      step_max = fmaxf(step_max, __shfl_xor(step_max, 16, WAVE));
      step_max = fmaxf(step_max, __shfl_xor(step_max, 32, WAVE));
      step_max *= scale_log2;                                        // scale > 0: the maximum stays the maximum
      const float m_new = fmaxf(acc.m[s], step_max);
      const float m_safe = m_new == -INFINITY ? 0.f : m_new;       // nothing visible yet
      const float correction = __builtin_amdgcn_exp2f(acc.m[s] - m_safe);
      acc.m[s] = m_new;
      mfma_bf16x8 p_frag;
      float sum = 0.f;
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const float p = __builtin_amdgcn_exp2f(fmaf(score[t][i], scale_log2, -m_safe));
          sum += p;
          p_frag[4 * t + i] = (bf16_t)p;
        }
      acc.l[s] = acc.l[s] * correction + sum;
#pragma unroll
      for (int dt = 0; dt < DH / 16; ++dt) {
#pragma unroll
        for (int i = 0; i < 4; ++i) acc.o[s][dt][i] *= correction;
        acc.o[s][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(f.v[st][dt], p_frag, acc.o[s][dt], 0, 0, 0);
      }
    }
  }
}

// Keys [key_lo, key_hi): key_lo a multiple of 4; every key < key_hi is in the cache.
// q_frag[s][kk]: lane (q, n) holds Q[column n of set s][dims 32*kk + 8q .. +8].
// col_pos[s]: the position of lane's column n in set s (its last visible key), or -1 for a
// column that holds no query.  window: 0 = none.  STEPS: 32-key steps whose loads are all
// requested before the first is used.  PIPELINED: the loads of the next STEPS steps are
// requested before the current ones are worked on (twice the fragment registers), for callers
// with long runs; a caller whose run is one round of STEPS steps gains nothing from it.
// min_pos / max_pos: the smallest and largest position among the columns of the wave, when all
// of them hold queries and the caller knows (the same value in every lane), else -1.
template <int DH, int NSET, int STEPS, bool PIPELINED = false>
__device__ __forceinline__ void attend_keys(AttnAccumulator<DH, NSET>& acc,
                                            const mfma_bf16x8 (&q_frag)[NSET][DH / 32],
                                            const int (&col_pos)[NSET], int window, float scale, int key_lo,
                                            int key_hi, const AttnCache& cache, int min_pos = -1, int max_pos = -1) {
  const int last_key = key_hi - 1;
  constexpr int ROUND = 32 * STEPS;
  if (PIPELINED) {
    // the next round is always asked for, also past the end of the run (its keys are clamped to
    // the last one and never used): a condition around the loads would cost a wait
    AttnFragments<DH, STEPS> even, odd;
    attn_load<DH, STEPS>(even, key_lo, last_key, cache);
    for (int k00 = key_lo; k00 < key_hi; k00 += 2 * ROUND) {
      attn_load<DH, STEPS>(odd, k00 + ROUND, last_key, cache);
      attn_compute<DH, NSET, STEPS>(acc, even, q_frag, col_pos, window, scale, k00, key_hi);
      attn_load<DH, STEPS>(even, k00 + 2 * ROUND, last_key, cache);
      if (k00 + ROUND < key_hi) attn_compute<DH, NSET, STEPS>(acc, odd, q_frag, col_pos, window, scale, k00 + ROUND, key_hi);
    }
  } else {
    // rounds all of whose keys every column of the wave sees run without masks, in a loop of
    // their own; the rest (the diagonal, a window's edge, the end of the run) with them
    int open_hi = key_lo;
    if (min_pos >= 0 && (window <= 0 || key_lo >= max_pos - window + 1))
      open_hi = key_lo + max(0, (min(min_pos + 1, key_hi) - key_lo) / ROUND) * ROUND;
    for (int k00 = key_lo; k00 < open_hi; k00 += ROUND) {
      AttnFragments<DH, STEPS> f;
      attn_load<DH, STEPS>(f, k00, last_key, cache);
      attn_compute<DH, NSET, STEPS, false>(acc, f, q_frag, col_pos, window, scale, k00, key_hi);
    }
    for (int k00 = open_hi; k00 < key_hi; k00 += ROUND) {
      AttnFragments<DH, STEPS> f;
      attn_load<DH, STEPS>(f, k00, last_key, cache);
      attn_compute<DH, NSET, STEPS, true>(acc, f, q_frag, col_pos, window, scale, k00, key_hi);
    }
  }
}

// The normalizer of lane's column: the shares of the four lanes (q = 0..3) that hold it.
template <int DH, int NSET>
__device__ __forceinline__ float attn_normalizer(const AttnAccumulator<DH, NSET>& acc, int s) {
  float l = acc.l[s];
  l += __shfl_xor(l, 16, WAVE);
  l += __shfl_xor(l, 32, WAVE);
  return l;
}
