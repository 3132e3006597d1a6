// Entry points that allocate nothing.
//
// These have no counterpart in the reference.  They are for callers that cannot allocate device memory:
// code that runs under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Such an
// entry point is a variant of an existing one whose kernels need device memory beyond their inputs and
// outputs (partial results of workgroups that a second kernel merges); instead of a workspace argument it
// uses an array of fixed size that lives in the library's own device image.
//
// Rules of use:
//   * the caller still passes every input and output; the stream must belong to the device that is
//     current in the calling thread;
//   * every GPU the library runs on holds its own copy of the array (MI_STATIC_SCRATCH_BYTES, until the
//     process ends); a call whose partial results do not fit returns ERR_UNSUPPORTED_SIZE (-2) with
//     nothing launched;
//   * all calls on one GPU share that GPU's array, and the array keeps the last call's contents.  Nothing
//     in it has to start at zero: the merge reads only what the same call has written.  Calls that overlap
//     on one GPU (two streams, two threads) race: serialize them.
//   * no hipMalloc, hipFree or allocating library routine is called, on the first call or later.
#pragma once
#include <hip/hip_runtime.h>

#define MI_STATIC_SCRATCH_BYTES (8u << 20)

#ifdef __cplusplus
extern "C" {
#endif

// mi_decode_attention (split-context attention of single-token queries over the paged cache, bfloat16)
// with the partial outputs [T, Hq, splits, dh] and their (max, sum) [T, Hq, splits, 2] kept in the static
// array: T * Hq * splits * (dh + 2) floats (each part rounded up to 256 bytes) must fit MI_STATIC_SCRATCH_BYTES.
// Same arguments, same kernels, same result as mi_decode_attention.
int mi_decode_attention_static(const void* q, long q_ld, int T, int Hq, int Hkv, int dh, const void* k_base,
                               const void* v_base, long page_stride, int page_size, const int* block_tables,
                               int max_pages, const int* lane_of_token, const int* positions, float scale,
                               int window, int split_keys, int splits, void* out, long out_ld,
                               hipStream_t stream);

// The size of the static array in bytes.
long mi_static_scratch_bytes(void);

#ifdef __cplusplus
}
#endif
