// bfloat16 matrix products on the matrix cores (MFMA), 32-bit accumulation:
//   C[M,N] (+)= A[M,K] . W[N,K]^T,   W in the nn.Linear layout [out, in]
// (crates/glassbox-core/src/kernels.rs:381,586).  Both operands are contiguous along k, which
// is the layout MFMA operands want: every lane loads 8 consecutive k as one 16-byte word.
//
// Two kernels:
//  * tiled  (M > 64, prompt portions): 128x128 tile per workgroup of 4 waves, each wave a 64x64
//    block of 2x2 v_mfma_f32_32x32x16_bf16 tiles, operands staged through LDS in k-steps of 32
//    with two buffers.
//  * skinny (M <= 64, decoding): bound by reading W once.  A workgroup owns 16 rows of W; its 4
//    waves take interleaved 64-wide k blocks, stream W straight from memory into MFMA operands
//    (v_mfma_f32_16x16x32_bf16, W as the A operand so that the 16 rows fill the tile) and combine
//    through LDS in a fixed order.
// In both, every output cell is summed in an order fixed by (K, kernel) alone, not by M or by
// the cell's neighbours.  C is bfloat16 or float32; accumulation (+=) is into float32.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

template <typename CT> __device__ __forceinline__ void store_c(CT* c, float v, int accumulate);
template <> __device__ __forceinline__ void store_c<float>(float* c, float v, int accumulate) { *c = accumulate ? *c + v : v; }
template <> __device__ __forceinline__ void store_c<bf16>(bf16* c, float v, int) { *c = (bf16)v; }

// ------------------------------------------------------------------------- tiled
constexpr int TBM = 128, TBN = 128, TBK = 32, TLD = TBK + 8;  // LDS row stride in elements (80 bytes)

template <typename CT>
__global__ __launch_bounds__(256) void gemm_tiled_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w,
                                                         int ldw, CT* __restrict__ c, int ldc, int M, int N, int K,
                                                         int accumulate) {
  __shared__ __attribute__((aligned(16))) bf16 As[2][TBM][TLD];
  __shared__ __attribute__((aligned(16))) bf16 Ws[2][TBN][TLD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;  // 2 x 2 waves, 64 x 64 each
  const int m0 = blockIdx.y * TBM, n0 = blockIdx.x * TBN;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // each thread moves two 16-byte chunks of A and two of W per k-step
  bf16x8 ga[2], gw[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ch = tid + 256 * j, row = ch / 4, kc = (ch % 4) * 8;
      const int gk = k0 + kc;
      ga[j] = (m0 + row < M && gk < K) ? load8(a + (size_t)(m0 + row) * lda + gk) : zero8();
      gw[j] = (n0 + row < N && gk < K) ? load8(w + (size_t)(n0 + row) * ldw + gk) : zero8();
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int ch = tid + 256 * j, row = ch / 4, kc = (ch % 4) * 8;
      *reinterpret_cast<bf16x8*>(&As[buf][row][kc]) = ga[j];
      *reinterpret_cast<bf16x8*>(&Ws[buf][row][kc]) = gw[j];
    }
  };

  fetch(0);
  stash(0);
  __syncthreads();
  const int steps = (K + TBK - 1) / TBK;
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) fetch((s + 1) * TBK);
#pragma unroll
    for (int ks = 0; ks < TBK / 16; ++ks) {
      bf16x8 fa[2], fw[2];
      const int kk = ks * 16 + 8 * (lane / 32);
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = *reinterpret_cast<const bf16x8*>(&As[buf][wm * 64 + i * 32 + lane % 32][kk]);
#pragma unroll
      for (int j = 0; j < 2; ++j) fw[j] = *reinterpret_cast<const bf16x8*>(&Ws[buf][wn * 64 + j * 32 + lane % 32][kk]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[i], fw[j], acc[i][j], 0, 0, 0);
    }
    if (s + 1 < steps) stash(buf ^ 1);
    __syncthreads();
  }

  // accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int gn = n0 + wn * 64 + j * 32 + lane % 32;
      if (gn >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm * 64 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (gm < M) store_c<CT>(c + (size_t)gm * ldc + gn, acc[i][j][r], accumulate);
      }
    }
}

// ------------------------------------------------------------------------ skinny
// MT = number of 16-wide column blocks of A's rows (M <= 16*MT).
template <int MT, typename CT>
__global__ __launch_bounds__(256) void gemm_skinny_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w,
                                                          int ldw, CT* __restrict__ c, int ldc, int M, int N, int K,
                                                          int accumulate) {
  __shared__ float part[4][MT][64][4];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const int n0 = blockIdx.x * 16;
  const int row = n0 + r;
  const bool row_ok = row < N;
  const bf16* wrow = w + (size_t)(row_ok ? row : 0) * ldw;

  f32x4 acc[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[t][e] = 0.f;

  // wave `wave` takes the 64-wide k blocks wave, wave+4, ...; inside a block lane group q holds
  // k = 16q .. 16q+15 as two operands of 8 (the same split for W and for A, so the products pair up)
#pragma unroll 4
  for (int kb = wave * 64; kb < K; kb += 256) {
    const int k = kb + q * 16;
    bf16x8 w0 = (row_ok && k < K) ? load8(wrow + k) : zero8();
    bf16x8 w1 = (row_ok && k + 8 < K) ? load8(wrow + k + 8) : zero8();
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + r;
      const bf16* arow = a + (size_t)(m < M ? m : 0) * lda;
      bf16x8 x0 = (m < M && k < K) ? load8(arow + k) : zero8();
      bf16x8 x1 = (m < M && k + 8 < K) ? load8(arow + k + 8) : zero8();
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w0, x0, acc[t], 0, 0, 0);
      acc[t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(w1, x1, acc[t], 0, 0, 0);
    }
  }
#pragma unroll
  for (int t = 0; t < MT; ++t)
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave][t][lane][e] = acc[t][e];
  __syncthreads();
  // D[n, m]: lane holds column m = lane%16 and rows n = 4*(lane/16) + e.  256 threads share the
  // MT*64*4 cells; the four waves' partial sums are added in wave order.
  for (int cell = tid; cell < MT * 64 * 4; cell += 256) {
    const int t = cell / 256, l = (cell / 4) % 64, e = cell % 4;
    const float v = ((part[0][t][l][e] + part[1][t][l][e]) + part[2][t][l][e]) + part[3][t][l][e];
    const int m = t * 16 + l % 16, n = n0 + 4 * (l / 16) + e;
    if (m < M && n < N) store_c<CT>(c + (size_t)m * ldc + n, v, accumulate);
  }
}

template <typename CT>
int launch(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, int accumulate,
           hipStream_t stream) {
  if (M <= 64) {
    const dim3 grid((N + 15) / 16), block(256);
    const int mt = (M + 15) / 16;
    if (mt == 1) hipLaunchKernelGGL((gemm_skinny_kernel<1, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
    else if (mt == 2) hipLaunchKernelGGL((gemm_skinny_kernel<2, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
    else if (mt == 3) hipLaunchKernelGGL((gemm_skinny_kernel<3, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
    else hipLaunchKernelGGL((gemm_skinny_kernel<4, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
  } else {
    const dim3 grid((N + TBN - 1) / TBN, (M + TBM - 1) / TBM), block(256);
    if (grid.y > 65535) return fail("gemm_bf16: M=%d needs more than 65535 row tiles", M);
    hipLaunchKernelGGL(gemm_tiled_kernel<CT>, grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
  }
  return launched("gemm_bf16");
}

}  // namespace

extern "C" int gb_gemm_bf16(const void* a, int lda, const void* w, int ldw, void* c, int ldc, int c_dtype, int M, int N,
                            int K, int accumulate, hipStream_t stream) {
  GB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  GB_REQUIRE(K % 8 == 0, "gemm_bf16: the inner size K=%d must be a multiple of 8 (16-byte operand loads)", K);
  GB_REQUIRE(lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: row strides (%d, %d) must be multiples of 8 elements", lda, ldw);
  GB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_bf16: a leading dimension is shorter than its row");
  GB_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  GB_REQUIRE(!accumulate || c_dtype == kF32, "gemm_bf16: accumulation is into a float32 result");
  if (M == 0) return 0;
  if (c_dtype == kF32) return launch<float>((const bf16*)a, lda, (const bf16*)w, ldw, (float*)c, ldc, M, N, K, accumulate, stream);
  if (c_dtype == kBF16) return launch<bf16>((const bf16*)a, lda, (const bf16*)w, ldw, (bf16*)c, ldc, M, N, K, accumulate, stream);
  return fail("gemm_bf16: unknown result dtype %d", c_dtype);
}
