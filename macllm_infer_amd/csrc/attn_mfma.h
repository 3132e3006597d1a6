// Attention over the paged cache on the matrix cores (bfloat16, v_mfma_f32_16x16x32_bf16),
// one wavefront at a time, shared by the prefill kernel (columns = 16 queries of one head)
// and the decode kernel (columns = the query heads of one kv head).
//
// A wave works on NSET sets of 16 columns that read the same kv head, and walks a run of keys
// 32 at a time:
//   scores   S^T[key, col] = K[key, :] . Q[col, :]     A = K (16 keys x 32 dims, contiguous in
//            dims), B = Q^T (contiguous in dims): no transposes; the result lands with lane
//            (q, n) holding keys 4q..4q+3 of each 16-key tile for column n;
//   softmax  online, per column, in float32: running maximum and normalizer, the accumulator
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

template <int DH, int NSET>
struct AttnAccumulator {
  float m[NSET];                       // running maximum of this lane's column in each set
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

// Keys [key_lo, key_hi): key_lo a multiple of 4; every key < key_hi is in the cache.
// q_frag[s][kk]: lane (q, n) holds Q[column n of set s][dims 32*kk + 8q .. +8].
// col_pos[s]: the position of lane's column n in set s (its last visible key), or -1 for a
// column that holds no query.  window: 0 = none.  STEPS: 32-key steps whose loads are all
// requested before the first is used (more loads in flight for latency-bound callers).
template <int DH, int NSET, int STEPS>
__device__ __forceinline__ void attend_keys(AttnAccumulator<DH, NSET>& acc,
                                            const mfma_bf16x8 (&q_frag)[NSET][DH / 32],
                                            const int (&col_pos)[NSET], int window, float scale, int key_lo,
                                            int key_hi, const AttnCache& cache) {
  const int lane = threadIdx.x & (WAVE - 1);
  const int q = lane / 16;
  const int r = lane % 16;
  const int last_key = key_hi - 1;
  for (int k00 = key_lo; k00 < key_hi; k00 += 32 * STEPS) {
    // ---- loads: K rows of two 16-key tiles per step, V^T columns of the same 32 keys
    mfma_bf16x8 k_frag[STEPS][2][DH / 32];
    mfma_bf16x8 v_frag[STEPS][DH / 16];
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
        for (int kk = 0; kk < DH / 32; ++kk)
          k_frag[st][t][kk] = *reinterpret_cast<const mfma_bf16x8*>(row + 32 * kk);
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
          for (int j = 0; j < 4; ++j) v_frag[st][dt][4 * t + j] = part[j];
        }
      }
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
      const int k0 = k00 + 32 * st;
      if (k0 >= key_hi) break;
      if (k0 + 32 > key_hi) {
        // the run ends inside this step: cells past it were never written; keep them out of the product
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            if (k0 + 16 * t + 4 * q + j > last_key) {
#pragma unroll
              for (int dt = 0; dt < DH / 16; ++dt) v_frag[st][dt][4 * t + j] = (bf16_t)0.f;
            }
      }
      // ---- per set of columns: scores, softmax step, values
#pragma unroll
      for (int s = 0; s < NSET; ++s) {
        mfma_floatx4 score[2];
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          score[t] = mfma_floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int kk = 0; kk < DH / 32; ++kk)
            score[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(k_frag[st][t][kk], q_frag[s][kk], score[t], 0, 0, 0);
        }
        const int position = col_pos[s];
        const int first_visible = window > 0 ? position - window + 1 : 0;
        float step_max = -INFINITY;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const int key = k0 + 16 * t + 4 * q + i;
            const bool visible = key <= position && key >= first_visible && key <= last_key;
            score[t][i] = visible ? score[t][i] * scale : -INFINITY;
            step_max = fmaxf(step_max, score[t][i]);
          }
        step_max = fmaxf(step_max, __shfl_xor(step_max, 16, WAVE));
        step_max = fmaxf(step_max, __shfl_xor(step_max, 32, WAVE));
        const float m_new = fmaxf(acc.m[s], step_max);
        const float m_safe = m_new == -INFINITY ? 0.f : m_new;       // nothing visible yet
        const float correction = __expf(acc.m[s] - m_safe);
        acc.m[s] = m_new;
        mfma_bf16x8 p_frag;
        float sum = 0.f;
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            const float p = __expf(score[t][i] - m_safe);
            sum += p;
            p_frag[4 * t + i] = (bf16_t)p;
          }
        acc.l[s] = acc.l[s] * correction + sum;
#pragma unroll
        for (int dt = 0; dt < DH / 16; ++dt) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc.o[s][dt][i] *= correction;
          acc.o[s][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(v_frag[st][dt], p_frag, acc.o[s][dt], 0, 0, 0);
        }
      }
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
