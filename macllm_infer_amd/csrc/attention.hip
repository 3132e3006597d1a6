// Rotary position encoding fused with the write of K and V into cache pages, and
// attention over the paged cache.
//
// Cache layout of one paged group: [page, layer, 2 (K,V), kv_head, token_in_page, head_dim].
// Entry points get the base pointers of one layer's K and V inside page 0 and the
// stride between pages, so  K(page, kvh, off) = k_base + page*page_stride + (kvh*page_size + off)*dh.
// (The reference addresses its pages the same way: crates/macllm-kv/src/cache.rs:558-566,
// crates/macllm-kernels/src/metal/paged_decode.metal:109-113.)
#include "common.h"

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
      v_base[page * page_stride + ((long)kvh * page_size + offset) * dh + i] = v[item];
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
// One wavefront per (token, query head).  Keys are taken 64 at a time: lane i scores key i
// (full dot product over dh from its own cache row), the wave keeps the running maximum
// and normalizer in float32 (online softmax), and for the value product lane i owns output
// dims i, i+64, ...  Works for any head_dim <= 256, any page size, any group size.
//   s = q.k * scale;  visible keys: position <= query position, and
//   query - key < window when window > 0 (reference: src/decoder.rs:4515-4532);
//   softmax in float32 (reference: src/decoder.rs:4665-4667).
#define ATT_MAX_DH 256

template <typename T, bool FAST_EXP>
__global__ void __launch_bounds__(WAVE)
paged_attention_kernel(const T* __restrict__ q, long q_ld, int Hq, int Hkv, int dh,
                       const T* __restrict__ k_base, const T* __restrict__ v_base, long page_stride,
                       int page_size, const int* __restrict__ block_tables, int max_pages,
                       const int* __restrict__ lane_of_token, const int* __restrict__ positions, float scale,
                       int window, T* __restrict__ out, long out_ld) {
  __shared__ float q_shared[ATT_MAX_DH];
  __shared__ float p_shared[WAVE];
  __shared__ long row_shared[WAVE];
  const long token = blockIdx.x;
  const int head = blockIdx.y;
  const int kvh = head / (Hq / Hkv);
  const int lane = threadIdx.x;
  const int request = lane_of_token[token];
  const int query_position = positions[token];
  const int* table = block_tables + (long)request * max_pages;
  const T* q_row = q + token * q_ld + (long)head * dh;
  for (int i = lane; i < dh; i += WAVE) q_shared[i] = to_float(q_row[i]);
  __syncthreads();

  int first_key = 0;
  if (window > 0 && query_position - window + 1 > 0) first_key = query_position - window + 1;
  const int last_key = query_position;     // inclusive

  float running_max = -INFINITY;
  float running_sum = 0.f;
  float acc[ATT_MAX_DH / WAVE];
#pragma unroll
  for (int i = 0; i < ATT_MAX_DH / WAVE; ++i) acc[i] = 0.f;

  for (int base = first_key; base <= last_key; base += WAVE) {
    const int key = base + lane;
    float score = -INFINITY;
    long row_offset = 0;
    if (key <= last_key) {
      const int page = table[key / page_size];
      const int offset = key % page_size;
      row_offset = (long)page * page_stride + ((long)kvh * page_size + offset) * dh;
      const T* k_row = k_base + row_offset;
      float dot = 0.f;
      for (int i = 0; i < dh; ++i) dot += q_shared[i] * to_float(k_row[i]);
      score = dot * scale;
    }
    const float block_max = wave_max(score);
    const float new_max = fmaxf(running_max, block_max);
    const float correction = FAST_EXP ? __expf(running_max - new_max) : expf(running_max - new_max);
    const float p = (key <= last_key) ? (FAST_EXP ? __expf(score - new_max) : expf(score - new_max)) : 0.f;
    running_sum = running_sum * correction + wave_sum(p);
    running_max = new_max;
    __syncthreads();
    p_shared[lane] = p;
    row_shared[lane] = row_offset;
    __syncthreads();
    const int valid = min(WAVE, last_key - base + 1);
#pragma unroll
    for (int i = 0; i < ATT_MAX_DH / WAVE; ++i) {
      const int dim = lane + i * WAVE;
      if (dim < dh) {
        float sum = acc[i] * correction;
        for (int j = 0; j < valid; ++j) sum += p_shared[j] * to_float(v_base[row_shared[j] + dim]);
        acc[i] = sum;
      }
    }
  }
  T* o = out + token * out_ld + (long)head * dh;
#pragma unroll
  for (int i = 0; i < ATT_MAX_DH / WAVE; ++i) {
    const int dim = lane + i * WAVE;
    if (dim < dh) o[dim] = from_float<T>(acc[i] / running_sum);
  }
}

extern "C" int mi_paged_attention(const void* q, int dtype, long q_ld, int T, int Hq, int Hkv, int dh,
                                  const void* k_base, const void* v_base, long page_stride, int page_size,
                                  const int* block_tables, int max_pages, const int* lane_of_token,
                                  const int* positions, float scale, int window, void* out, long out_ld,
                                  hipStream_t stream) {
  if (T <= 0 || Hq <= 0 || Hkv <= 0 || Hq % Hkv != 0 || dh <= 0 || page_size <= 0 || max_pages <= 0)
    return ERR_BAD_ARGUMENT;
  if (dh > ATT_MAX_DH) return ERR_UNSUPPORTED_SIZE;
  if (Hq > 65535) return ERR_UNSUPPORTED_SIZE;
  const dim3 grid(T, Hq);
  if (dtype == DT_F32)
    paged_attention_kernel<float, false><<<grid, WAVE, 0, stream>>>(
        (const float*)q, q_ld, Hq, Hkv, dh, (const float*)k_base, (const float*)v_base, page_stride, page_size,
        block_tables, max_pages, lane_of_token, positions, scale, window, (float*)out, out_ld);
  else if (dtype == DT_BF16)
    paged_attention_kernel<bf16_t, true><<<grid, WAVE, 0, stream>>>(
        (const bf16_t*)q, q_ld, Hq, Hkv, dh, (const bf16_t*)k_base, (const bf16_t*)v_base, page_stride,
        page_size, block_tables, max_pages, lane_of_token, positions, scale, window, (bf16_t*)out, out_ld);
  else
    return ERR_BAD_ARGUMENT;
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
