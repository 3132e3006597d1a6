// Matrix products of the float32 path: out[M, N] = x[M, K] . W[N, K]^T (+ bias[N]), with float32
// operands, products and sums throughout (v_mfma_f32_16x16x4_f32 multiplies and adds in float32; no
// reduced-precision matrix mode).
//
// One kernel serves a decode step of a few rows and a prompt portion of thousands: a workgroup owns
// NT tiles of 16 output features and MT tiles of 16 rows, its four waves split K into four contiguous
// runs of 16-wide chunks, and their partial tiles are added through LDS in the order of the waves.  The
// order in which an output element is summed depends on K alone (which chunks a wave owns, the four
// products of a chunk in turn, wave 0 to 3), never on M, on the tiling or on the rows beside it: a
// row's result is bit for bit the same alone, in a small step and in a large one.
//
// A step of up to 16 rows is bound by reading W once: every wave keeps eight 1 KiB fragments of it in
// flight.  A large M re-reads x once per 64 features and W once per 64 rows, from the caches.
#include "common.h"

typedef float floatx4 __attribute__((ext_vector_type(4)));

#define GF_WAVES 4
#define GF_THREADS (GF_WAVES * WAVE)

// four consecutive k of one row; VEC: one 16-byte load (K, the leading dimension and the base are
// multiples of 4 floats); otherwise four loads, each checked against K.  A k at or past K gives zero.
template <bool VEC>
__device__ __forceinline__ floatx4 load_k4(const float* row, int k, int K) {
  if (VEC) {
    const floatx4 value = *reinterpret_cast<const floatx4*>(row + min(k, K - 4));
    return k < K ? value : floatx4{0.f, 0.f, 0.f, 0.f};
  }
  floatx4 value;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const float element = row[min(k + j, K - 1)];
    value[j] = k + j < K ? element : 0.f;
  }
  return value;
}

template <int MT, int NT, int DEPTH, bool VEC>
__global__ void __launch_bounds__(GF_THREADS)
gemm_f32_kernel(const float* __restrict__ x, long ldx, const float* __restrict__ W, long ldw,
                const float* __restrict__ bias, float* __restrict__ out, long ldo, int M, int N, int K) {
  __shared__ float red[GF_WAVES][MT][256];
  const int tid = threadIdx.x;
  const int lane = tid & (WAVE - 1);
  const int wave = tid / WAVE;
  const int q = lane / 16;
  const int r = lane % 16;
  const long n0 = (long)blockIdx.x * 16 * NT;
  const long m0 = (long)blockIdx.y * 16 * MT;
  const float* w_row[NT];
  const float* x_row[MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) w_row[nt] = W + min(n0 + 16 * nt + r, (long)N - 1) * ldw;
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) x_row[mt] = x + min(m0 + 16 * mt + r, (long)M - 1) * ldx;

  const int chunks = (K + 15) / 16;
  const int per_wave = (chunks + GF_WAVES - 1) / GF_WAVES;
  const int first_chunk = wave * per_wave;
  const int iterations = max(0, min(per_wave, chunks - first_chunk));

  floatx4 acc[NT][MT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[nt][mt] = floatx4{0.f, 0.f, 0.f, 0.f};

  // DEPTH chunks are asked for before the first is used; no branch between the loads (a chunk past
  // the wave's run reads the run's last one again and is not multiplied)
  for (int first = 0; first < iterations; first += DEPTH) {
    floatx4 a[DEPTH][NT], b[DEPTH][MT];
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const int k = (first_chunk + min(first + j, iterations - 1)) * 16 + 4 * q;
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) a[j][nt] = load_k4<VEC>(w_row[nt], k, K);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) b[j][mt] = load_k4<VEC>(x_row[mt], k, K);
    }
    // a step of few rows waits for its weights: every load of the round is asked for before its first product (left
    // to itself the scheduler moves each load down to the product that uses it and waits for it there, one round
    // trip to memory after the other; the tiles of many rows, which wait for their products, are better left to it)
    if (NT == 1) __builtin_amdgcn_sched_barrier(0);
    // no branch around the products either (under one the compiler waits for each load where it is used,
    // one at a time): a chunk past the end is multiplied as zeros
#pragma unroll
    for (int j = 0; j < DEPTH; ++j) {
      const bool live = first + j < iterations;
      const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
      floatx4 weights[NT], rows[MT];
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) weights[nt] = live ? a[j][nt] : zero;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) rows[mt] = live ? b[j][mt] : zero;
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[nt][mt] = __builtin_amdgcn_mfma_f32_16x16x4f32(weights[nt][i], rows[mt][i], acc[nt][mt], 0, 0, 0);
    }
  }

  // the waves' partial tiles, added in the order of the waves, one tile of 16 features after the other
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) {
    if (nt > 0) __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int i = 0; i < 4; ++i) red[wave][mt][i * 64 + lane] = acc[nt][mt][i];
    __syncthreads();
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      // element tid of the tile: feature 4 (l / 16) + i, row l % 16, stored at i * 64 + l
      const int i = tid / 64;
      const int l = tid % 64;
      float value = red[0][mt][tid];
#pragma unroll
      for (int w = 1; w < GF_WAVES; ++w) value += red[w][mt][tid];
      const long n = n0 + 16 * nt + 4 * (l / 16) + i;
      const long m = m0 + 16 * mt + (l % 16);
      if (n < N && m < M) out[m * ldo + n] = bias ? value + bias[n] : value;
    }
  }
}

template <int MT, int NT, int DEPTH>
static void launch_gemm_f32(bool vec, dim3 grid, hipStream_t stream, const float* x, long ldx, const float* W,
                            long ldw, const float* bias, float* out, long ldo, int M, int N, int K) {
  if (vec) gemm_f32_kernel<MT, NT, DEPTH, true><<<grid, GF_THREADS, 0, stream>>>(x, ldx, W, ldw, bias, out, ldo, M, N, K);
  else gemm_f32_kernel<MT, NT, DEPTH, false><<<grid, GF_THREADS, 0, stream>>>(x, ldx, W, ldw, bias, out, ldo, M, N, K);
}

extern "C" int mi_gemm_f32(const float* x, long ldx, const float* W, long ldw, const float* bias, float* out,
                           long ldo, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldo < N) return ERR_BAD_ARGUMENT;
  const bool vec = K % 4 == 0 && ldx % 4 == 0 && ldw % 4 == 0 && ((unsigned long long)x % 16) == 0 &&
                   ((unsigned long long)W % 16) == 0;
  // rows and features of a workgroup: one tile of features while the step is small (W is read once, by as
  // many workgroups as there are tiles of it); 64 x 64 for many rows (x and W come from the caches)
  const int row_tiles = M <= 16 ? 1 : M <= 32 ? 2 : 4;
  const int feature_tiles = M <= 64 ? 1 : 4;
  const long blocks_x = ((long)N + 16 * feature_tiles - 1) / (16 * feature_tiles);
  const long blocks_y = ((long)M + 16 * row_tiles - 1) / (16 * row_tiles);
  if (blocks_y > 65535 || blocks_x > 0x7fffffffL) return ERR_UNSUPPORTED_SIZE;
  const dim3 grid((unsigned)blocks_x, (unsigned)blocks_y);
  if (feature_tiles == 4) launch_gemm_f32<4, 4, 2>(vec, grid, stream, x, ldx, W, ldw, bias, out, ldo, M, N, K);
  else if (row_tiles == 4) launch_gemm_f32<4, 1, 4>(vec, grid, stream, x, ldx, W, ldw, bias, out, ldo, M, N, K);
  else if (row_tiles == 2) launch_gemm_f32<2, 1, 4>(vec, grid, stream, x, ldx, W, ldw, bias, out, ldo, M, N, K);
  else launch_gemm_f32<1, 1, 8>(vec, grid, stream, x, ldx, W, ldw, bias, out, ldo, M, N, K);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
