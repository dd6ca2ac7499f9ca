// 32-bit matrix product for the true 32-bit path: C[M,N] (+)= A[M,K] . W[N,K]^T with
// W in the nn.Linear layout [out, in] (crates/glassbox-core/src/kernels.rs:381,586).
// Plain fused multiply-adds in 32-bit, no matrix-core mode of reduced precision.  Every
// output cell is one dot product summed in ascending k by one thread, so its value does
// not depend on M, on the tile it falls in, or on what else is in the batch.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, int lda, const float* __restrict__ w,
                                                       int ldw, float* __restrict__ c, int ldc, int M, int N, int K,
                                                       int accumulate) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int j = 0; j < (BM * BK) / 256; ++j) {
      const int e = tid + 256 * j;
      const int r = e / BK, kk = e % BK;
      const int gm = m0 + r, gn = n0 + r, gk = k0 + kk;
      As[kk][r] = (gm < M && gk < K) ? a[(size_t)gm * lda + gk] : 0.f;
      Ws[kk][r] = (gn < N && gk < K) ? w[(size_t)gn * ldw + gk] : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float av[TM], wv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) av[i] = As[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) wv[j] = Ws[kk][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int gm = m0 + ty * TM + i;
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int gn = n0 + tx * TN + j;
      if (gn >= N) continue;
      float* dst = c + (size_t)gm * ldc + gn;
      *dst = accumulate ? *dst + acc[i][j] : acc[i][j];
    }
  }
}

}  // namespace

extern "C" int gb_gemm_f32(const float* a, int lda, const float* w, int ldw, float* c, int ldc, int M, int N, int K,
                           int accumulate, hipStream_t stream) {
  GB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  GB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: a leading dimension is shorter than its row (lda=%d ldw=%d ldc=%d)", lda, ldw, ldc);
  if (M == 0) return 0;
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  GB_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d needs more than 65535 row tiles", M);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
  return launched("gemm_f32");
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_gemm_f32)
