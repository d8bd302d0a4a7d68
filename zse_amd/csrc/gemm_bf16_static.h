// The bfloat16 matrix product for callers that cannot allocate device memory.
//
// This entry point has no counterpart in the reference.  It is for callers that cannot call
// hipMalloc: code under HIP graph capture, tight serving loops, harnesses that forbid
// allocation.  zk_gemm_bf16 takes a workspace from its caller for the partial sums of a
// product that splits K over blocks; zk_gemm_bf16_static keeps them in an array that is part
// of the library's device code instead, and neither allocates nor frees anything, on the
// device or through a library routine.  The caller still passes inputs and outputs.
//
//  * The array holds ZK_GEMM_STATIC_SCRATCH_BYTES on every GPU the library runs on, from the
//    library's first use on that GPU until the process ends.
//  * K is split exactly as zk_gemm_bf16 splits it when it is called with its standard workspace
//    (zk_gemm_bf16_workspace() bytes) and without ``parts``, so both give the same bits.  (With
//    ``parts`` a reader takes the partial sums over, and zk_gemm_bf16 may then split products
//    of up to 16 rows that it otherwise leaves whole; this entry point has no such reader.)
//    A shape whose partial sums
//    do not fit the array is refused with an error that names both sizes; nothing is launched.
//    Products of up to 64 rows always fit (their ranges times their padded width stay within
//    32768 columns: 64 x 32768 floats, twice that with a gate, are the array's 16 MiB);
//    products of more rows that split K fit while (tiles) x (ranges of K) x (4 bytes a tile
//    element) stays within the array.
//  * Every call on a GPU shares that GPU's array, which keeps the last call's contents.
//    Nothing in it has to start at zero (each plane of partial sums is written in full before
//    it is read, within one call), so calls need no clearing between them; but two calls
//    that overlap in time on one GPU (different streams, different threads) race on it.
//    Calls on one stream are ordered and safe.
//  * The array's address is looked up once per device, at zk_gemm_bf16_static_init() or at the
//    first call of zk_gemm_bf16_static on that device, with that device current.  A caller that
//    captures a graph calls zk_gemm_bf16_static_init() before the capture begins.
#pragma once
#include <cstddef>

#define ZK_GEMM_STATIC_SCRATCH_BYTES ((size_t)16 << 20)

extern "C" {

// Bytes of the static array.
size_t zk_gemm_bf16_static_bytes();

// Looks the array's address up for the current device (once; later calls return at once).
// 0 on success; on failure zk_last_error() says why.
int zk_gemm_bf16_static_init();

// C[M, N] = A[M, K] * W[N, K]^T, arguments as zk_gemm_bf16 without workspace and `parts`.
// 0 on success; non-zero with zk_last_error() set for a bad argument or a shape whose partial
// sums do not fit the array.
int zk_gemm_bf16_static(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32,
                        int M, int N, int K, int epi, float cap, int w_strip, void* stream);

}  // extern "C"
