// Plain matrix product C[M,N] = A[M,K] * W[N,K]^T with float accumulation,
// no matrix cores and no reduced precision: the 32-bit path's product and the
// twin that the tuned bf16 kernels are checked against.  Weights are
// [out, in] row-major as in the reference (orchestrator/kernels.py:1075-1126,
// a 32x32 shared-memory tile per block).  The sum over K runs in a fixed
// order for every output element, whatever M is, so a row's result does not
// depend on which other rows are in the batch.
#include "common.h"

#define GP_BM 64
#define GP_BN 64
#define GP_BK 16

template <typename TA, typename TC>
__global__ __launch_bounds__(256) void gemm_plain_kernel(const TA* __restrict__ A, int lda,
                                                         const TA* __restrict__ W,
                                                         TC* __restrict__ C, int ldc, int M, int N,
                                                         int K) {
  __shared__ float sA[GP_BK][GP_BM + 1];
  __shared__ float sW[GP_BK][GP_BN + 1];
  const int tx = threadIdx.x % 16, ty = threadIdx.x / 16;
  const int m0 = blockIdx.y * GP_BM, n0 = blockIdx.x * GP_BN;
  float acc[4][4] = {};
  for (int k0 = 0; k0 < K; k0 += GP_BK) {
    for (int i = threadIdx.x; i < GP_BM * GP_BK; i += 256) {
      const int r = i / GP_BK, c = i % GP_BK;
      const int m = m0 + r, n = n0 + r, k = k0 + c;
      sA[c][r] = (m < M && k < K) ? to_f32(A[(size_t)m * lda + k]) : 0.f;
      sW[c][r] = (n < N && k < K) ? to_f32(W[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < GP_BK; kk++) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; i++) a[i] = sA[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; j++) b[j] = sW[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = from_f32<TC>(acc[i][j]);
    }
  }
}

extern "C" int zk_gemm_plain(const void* A, int lda, const void* W, void* C, int ldc, int c_is_f32,
                             int M, int N, int K, void* stream) {
  ZK_REQUIRE(M >= 0 && N > 0 && K > 0, "zk_gemm_plain: bad sizes");
  ZK_REQUIRE(lda >= K && ldc >= N, "zk_gemm_plain: leading dimensions too small");
  if (M == 0) return 0;
  dim3 grid((N + GP_BN - 1) / GP_BN, (M + GP_BM - 1) / GP_BM);
  ZK_REQUIRE(grid.y <= 65535, "zk_gemm_plain: too many rows");
  hipStream_t s = (hipStream_t)stream;
  if (c_is_f32)
    gemm_plain_kernel<act_t, float><<<grid, 256, 0, s>>>((const act_t*)A, lda, (const act_t*)W,
                                                         (float*)C, ldc, M, N, K);
  else
    gemm_plain_kernel<act_t, act_t><<<grid, 256, 0, s>>>((const act_t*)A, lda, (const act_t*)W,
                                                         (act_t*)C, ldc, M, N, K);
  return zk_launch_status("zk_gemm_plain");
}
