// Matrix products of the float32 path: out[M, N] = x[M, K] . W[N, K]^T (+ bias[N]),
// computed with float32 FMAs only (no reduced-precision matrix mode).
// Every output element is accumulated by one thread in ascending k, so a row's result
// does not depend on how many other rows are in the batch.
#include "common.h"

#define GEMM_BM 64
#define GEMM_BN 64
#define GEMM_BK 16

__global__ void __launch_bounds__(256)
gemm_f32_kernel(const float* __restrict__ x, long ldx, const float* __restrict__ W, long ldw,
                const float* __restrict__ bias, float* __restrict__ out, long ldo, int M, int N, int K) {
  __shared__ float xs[GEMM_BK][GEMM_BM + 4];
  __shared__ float ws[GEMM_BK][GEMM_BN + 4];
  const int tx = threadIdx.x & 15;
  const int ty = threadIdx.x >> 4;
  const long m0 = (long)blockIdx.y * GEMM_BM;
  const long n0 = (long)blockIdx.x * GEMM_BN;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GEMM_BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int index = threadIdx.x + i * 256;
      const int row = index >> 4;
      const int kk = index & 15;
      const long m = m0 + row;
      const long n = n0 + row;
      const int k = k0 + kk;
      xs[kk][row] = (m < M && k < K) ? x[m * ldx + k] : 0.f;
      ws[kk][row] = (n < N && k < K) ? W[n * ldw + k] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GEMM_BK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = xs[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const long m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long n = n0 + tx * 4 + j;
      if (n < N) out[m * ldo + n] = acc[i][j] + (bias ? bias[n] : 0.f);
    }
  }
}

extern "C" int mi_gemm_f32(const float* x, long ldx, const float* W, long ldw, const float* bias, float* out,
                           long ldo, int M, int N, int K, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || ldx < K || ldw < K || ldo < N) return ERR_BAD_ARGUMENT;
  const long blocks_y = ((long)M + GEMM_BM - 1) / GEMM_BM;
  if (blocks_y > 65535) return ERR_UNSUPPORTED_SIZE;
  const dim3 grid((N + GEMM_BN - 1) / GEMM_BN, (unsigned)blocks_y);
  gemm_f32_kernel<<<grid, 256, 0, stream>>>(x, ldx, W, ldw, bias, out, ldo, M, N, K);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
