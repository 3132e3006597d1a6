// What this GPU's memory delivers to the simplest kernels: a streaming read and a streaming
// read-modify-write of a large buffer, 16 bytes a lane a load, every workgroup walking the buffer with the
// stride of the whole grid.  The figures are the ceilings that the decode kernels (weights read once, state
// read and written once) are measured against; the published peak of the memory is above both.
#include "common.h"

#define MB_THREADS 256

__global__ void __launch_bounds__(MB_THREADS) stream_read_kernel(const uint4* __restrict__ data, long count,
                                                                 unsigned* __restrict__ sink) {
  const long stride = (long)gridDim.x * MB_THREADS;
  unsigned acc = 0;
  long i = (long)blockIdx.x * MB_THREADS + threadIdx.x;
  for (; i + 3 * stride < count; i += 4 * stride) {         // four loads in flight a lane
    const uint4 a = data[i], b = data[i + stride], c = data[i + 2 * stride], d = data[i + 3 * stride];
    acc ^= a.x ^ a.y ^ a.z ^ a.w ^ b.x ^ b.y ^ b.z ^ b.w ^ c.x ^ c.y ^ c.z ^ c.w ^ d.x ^ d.y ^ d.z ^ d.w;
  }
  for (; i < count; i += stride) {
    const uint4 a = data[i];
    acc ^= a.x ^ a.y ^ a.z ^ a.w;
  }
  if (acc == 0x9e3779b9u) sink[0] = acc;                    // keeps the loads; almost never taken
}

__global__ void __launch_bounds__(MB_THREADS) stream_rmw_kernel(float4* __restrict__ data, long count, float scale) {
  const long stride = (long)gridDim.x * MB_THREADS;
  long i = (long)blockIdx.x * MB_THREADS + threadIdx.x;
  for (; i + 3 * stride < count; i += 4 * stride) {
    float4 a = data[i], b = data[i + stride], c = data[i + 2 * stride], d = data[i + 3 * stride];
    a.x *= scale; a.y *= scale; a.z *= scale; a.w *= scale;
    b.x *= scale; b.y *= scale; b.z *= scale; b.w *= scale;
    c.x *= scale; c.y *= scale; c.z *= scale; c.w *= scale;
    d.x *= scale; d.y *= scale; d.z *= scale; d.w *= scale;
    data[i] = a; data[i + stride] = b; data[i + 2 * stride] = c; data[i + 3 * stride] = d;
  }
  for (; i < count; i += stride) {
    float4 a = data[i];
    a.x *= scale; a.y *= scale; a.z *= scale; a.w *= scale;
    data[i] = a;
  }
}

// Reads `bytes` (a multiple of 16, 16-byte aligned) once with `blocks` workgroups.
extern "C" int mi_stream_read(const void* data, long bytes, void* sink, int blocks, hipStream_t stream) {
  if (!data || !sink || bytes <= 0 || bytes % 16 != 0 || blocks <= 0 || ((uintptr_t)data % 16) != 0) return ERR_BAD_ARGUMENT;
  stream_read_kernel<<<blocks, MB_THREADS, 0, stream>>>((const uint4*)data, bytes / 16, (unsigned*)sink);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}

// Reads and writes `bytes` of float32 once (every value times `scale`) with `blocks` workgroups.
extern "C" int mi_stream_rmw(void* data, long bytes, float scale, int blocks, hipStream_t stream) {
  if (!data || bytes <= 0 || bytes % 16 != 0 || blocks <= 0 || ((uintptr_t)data % 16) != 0) return ERR_BAD_ARGUMENT;
  stream_rmw_kernel<<<blocks, MB_THREADS, 0, stream>>>((float4*)data, bytes / 16, scale);
  RETURN_IF_LAUNCH_FAILED();
  return 0;
}
