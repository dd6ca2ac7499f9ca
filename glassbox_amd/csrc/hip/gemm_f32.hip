// 32-bit matrix product for the true 32-bit path: C[M,N] (+)= A[M,K] . W[N,K]^T with
// W in the nn.Linear layout [out, in] (crates/glassbox-core/src/kernels.rs:381,586).
// Plain fused multiply-adds in 32-bit, no matrix-core mode of reduced precision.
//
// Every output cell is summed in one order, whatever kernel computes it and whatever else is
// in the batch: k is cut into slices of 64; a slice's products are added in ascending k by a
// chain of fused multiply-adds that starts from zero; the slices' sums are added in ascending
// order.  So a cell's bits do not depend on M, on the tile it falls in, or on which of the three
// kernels ran:
//
//  * tiled (any sizes): a 64 x 64 tile of C a workgroup, k in steps of 16 through LDS, a thread
//    4 x 4 cells; after every fourth step (a slice) the chain's sum goes into the cell's total.
//  * wide (prompts; rows of 16 bytes): a 128 x 64 tile a workgroup and 8 x 4 cells a thread, so
//    that a k-step's 32 multiply-adds of a thread stand against three 16-byte reads from LDS
//    where the tiled kernel has 16 against two; the next k-step's operands are on their way
//    from memory while this one is multiplied, and LDS holds two k-steps, one barrier a step.
//    (Tiles of 128 x 128 with 8 x 8 cells leave one wave a SIMD on square products of 2,048 and
//    were slower at every size measured.)
//  * skinny (M <= 64, rows of 16 bytes: a decode step, a short prompt portion): the tiled kernel
//    would start N / 64 workgroups that walk all of k one step behind the other.  Here a workgroup
//    owns 8 rows of W and every lane one (slice, row) pair: it asks for its 64 weights at once
//    (64 KB on their way a workgroup), runs the chain for each row of A, and the slices' sums
//    meet in LDS, where one thread a cell adds them in order.  N / 8 workgroups: one for every
//    compute unit already at 2,048 rows of W.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kSlice = 64;   // the summation order's slice of k: both kernels keep to it

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;
static_assert(kSlice % BK == 0, "a slice is whole steps of the tiled kernel");

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* __restrict__ a, int lda, const float* __restrict__ w,
                                                       int ldw, float* __restrict__ c, int ldc, int M, int N, int K,
                                                       int accumulate) {
  __shared__ float As[BK][BM + 4];
  __shared__ float Ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  float acc[TM][TN], total[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = total[i][j] = 0.f;

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
    if ((k0 + BK) % kSlice == 0 || k0 + BK >= K) {   // a slice ends: its sum joins the total
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
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
      *dst = accumulate ? *dst + total[i][j] : total[i][j];
    }
  }
}

// ---- wide: 128 x 64 of C a workgroup, 8 x 4 cells a thread, two k-steps in LDS ------------------------------
constexpr int WM = 128, WN = 64, WK = 16;
static_assert(kSlice % WK == 0, "a slice is whole steps of the wide kernel");

__global__ __launch_bounds__(256) void gemm_f32_wide_kernel(const float* __restrict__ a, int lda, const float* __restrict__ w,
                                                            int ldw, float* __restrict__ c, int ldc, int M, int N, int K,
                                                            int accumulate) {
  constexpr int NB = WN / 64, CN = 4 * NB;   // blocks of 64 columns, columns a thread
  __shared__ __attribute__((aligned(16))) float As[2][WK][WM + 4];
  __shared__ __attribute__((aligned(16))) float Ws[2][WK][WN + 4];
  const int tid = threadIdx.x;
  const int tx = tid % 16, ty = tid / 16;
  const int m0 = blockIdx.y * WM, n0 = blockIdx.x * WN;
  // a thread brings word lc of the k-step's four for rows lr and lr + 64 of the operands
  const int lr = tid / 4, lc = tid % 4;
  f32x4 pa[2], pw[NB];
  const f32x4 zero = {0.f, 0.f, 0.f, 0.f};
  auto fetch = [&](int k0) {
    const int gk = k0 + 4 * lc;   // K is whole words: a word is inside k or outside
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int gm = m0 + lr + 64 * h;
      pa[h] = (gm < M && gk < K) ? *reinterpret_cast<const f32x4*>(a + (size_t)gm * lda + gk) : zero;
    }
#pragma unroll
    for (int h = 0; h < NB; ++h) {
      const int gn = n0 + lr + 64 * h;
      pw[h] = (gn < N && gk < K) ? *reinterpret_cast<const f32x4*>(w + (size_t)gn * ldw + gk) : zero;
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
      for (int h = 0; h < 2; ++h) As[buf][4 * lc + i][lr + 64 * h] = pa[h][i];
#pragma unroll
      for (int h = 0; h < NB; ++h) Ws[buf][4 * lc + i][lr + 64 * h] = pw[h][i];
    }
  };
  // cells (ty*4 + i%4 + 64*(i/4), tx*4 + j%4 + 64*(j/4))
  float acc[8][CN], total[8][CN];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int j = 0; j < CN; ++j) acc[i][j] = total[i][j] = 0.f;

  const int steps = (K + WK - 1) / WK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    if (s + 1 < steps) fetch((s + 1) * WK);
#pragma unroll
    for (int kk = 0; kk < WK; ++kk) {
      float av[8], wv[CN];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(&As[buf][kk][ty * 4 + 64 * h]);
#pragma unroll
        for (int i = 0; i < 4; ++i) av[4 * h + i] = x[i];
      }
#pragma unroll
      for (int h = 0; h < NB; ++h) {
        const f32x4 x = *reinterpret_cast<const f32x4*>(&Ws[buf][kk][tx * 4 + 64 * h]);
#pragma unroll
        for (int i = 0; i < 4; ++i) wv[4 * h + i] = x[i];
      }
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < CN; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    if (((s + 1) * WK) % kSlice == 0 || s + 1 == steps) {   // a slice ends: its sum joins the total
#pragma unroll
      for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < CN; ++j) {
          total[i][j] += acc[i][j];
          acc[i][j] = 0.f;
        }
    }
    // the other half of LDS was last read a step ago, before the barrier that every thread has passed since
    if (s + 1 < steps) stash(buf ^ 1);
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int gm = m0 + ty * 4 + (i & 3) + 64 * (i >> 2);
    if (gm >= M) continue;
#pragma unroll
    for (int j = 0; j < CN; ++j) {
      const int gn = n0 + tx * 4 + (j & 3) + 64 * (j >> 2);
      if (gn >= N) continue;
      float* dst = c + (size_t)gm * ldc + gn;
      *dst = accumulate ? *dst + total[i][j] : total[i][j];
    }
  }
}

// the wide kernel from so many of its tiles on; below that the small tiles spread the work further
constexpr int kWideMinTiles = 64;

// ---- skinny: 8 rows of W a workgroup, a lane a (slice, row) pair ------------------------------------------
constexpr int SR = 8;             // rows of W a workgroup
constexpr int SG = 256 / SR;      // slices in flight a workgroup: one a lane group of SR lanes
constexpr int SV = kSlice / 4;    // 16-byte words a slice of one row

template <int MT>   // rows of A a pass (the step's rows go MT at a time)
__global__ __launch_bounds__(256) void gemm_f32_skinny_kernel(const float* __restrict__ a, int lda,
                                                              const float* __restrict__ w, int ldw,
                                                              float* __restrict__ c, int ldc, int M, int N, int K,
                                                              int accumulate) {
  __shared__ float part[SG][SR][MT];
  const int tid = threadIdx.x;
  const int r = tid % SR, sl = tid / SR;
  const int n = blockIdx.x * SR + r;
  const int slices = (K + kSlice - 1) / kSlice;
  // the thread that adds the slices of cell (row cm of the pass, column cr)
  const int cr = tid % SR, cm = tid / SR;

  for (int m0 = 0; m0 < M; m0 += MT) {
    float total = 0.f;
    for (int s0 = 0; s0 < slices; s0 += SG) {
      const int k0 = (s0 + sl) * kSlice;
      const bool live = n < N && k0 < K;
      f32x4 wv[SV];
#pragma unroll
      for (int i = 0; i < SV; ++i) {
        const int k = k0 + 4 * i;
        wv[i] = (live && k < K) ? *reinterpret_cast<const f32x4*>(w + (size_t)n * ldw + k) : f32x4{0.f, 0.f, 0.f, 0.f};
      }
      float acc[MT];
#pragma unroll
      for (int m = 0; m < MT; ++m) acc[m] = 0.f;
      if (live) {
#pragma unroll
        for (int i = 0; i < SV; ++i) {
          const int k = k0 + 4 * i;
          if (k < K) {
#pragma unroll
            for (int m = 0; m < MT; ++m) {
              if (m0 + m < M) {
                const f32x4 x = *reinterpret_cast<const f32x4*>(a + (size_t)(m0 + m) * lda + k);
                acc[m] = fmaf(x[0], wv[i][0], acc[m]);
                acc[m] = fmaf(x[1], wv[i][1], acc[m]);
                acc[m] = fmaf(x[2], wv[i][2], acc[m]);
                acc[m] = fmaf(x[3], wv[i][3], acc[m]);
              }
            }
          }
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) part[sl][r][m] = acc[m];
      __syncthreads();
      if (cm < MT) {
        const int count = min(SG, slices - s0);
        for (int s = 0; s < count; ++s) total += part[s][cr][cm];
      }
      __syncthreads();
    }
    const int gm = m0 + cm, gn = blockIdx.x * SR + cr;
    if (cm < MT && gm < M && gn < N) {
      float* dst = c + (size_t)gm * ldc + gn;
      *dst = accumulate ? *dst + total : total;
    }
  }
}

template <int MT>
void launch_skinny(const float* a, int lda, const float* w, int ldw, float* c, int ldc, int M, int N, int K,
                   int accumulate, hipStream_t stream) {
  static_assert(MT <= SG, "one thread a cell of a pass");
  hipLaunchKernelGGL(gemm_f32_skinny_kernel<MT>, dim3((N + SR - 1) / SR), dim3(256), 0, stream, a, lda, w, ldw, c, ldc, M, N,
                     K, accumulate);
}

constexpr int kSkinnyMaxRows = 64;

inline bool words_of_16_bytes(const void* p, int ld) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0 && ld % 4 == 0; }

}  // namespace

// which = 0: the kernel the sizes call for; 1: the tiled kernel; 2: the skinny kernel; 3: the wide kernel (the last
// two refused where they do not apply).  All give the same bits; tests compare them.
extern "C" int gb_gemm_f32_by(const float* a, int lda, const float* w, int ldw, float* c, int ldc, int M, int N, int K,
                              int accumulate, int which, hipStream_t stream) {
  GB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_f32: bad sizes M=%d N=%d K=%d", M, N, K);
  GB_REQUIRE(lda >= K && ldw >= K && ldc >= N, "gemm_f32: a leading dimension is shorter than its row (lda=%d ldw=%d ldc=%d)", lda, ldw, ldc);
  GB_REQUIRE(which >= 0 && which <= 3, "gemm_f32: no kernel %d", which);
  if (M == 0) return 0;
  const bool words = K % 4 == 0 && words_of_16_bytes(a, lda) && words_of_16_bytes(w, ldw);
  const bool skinny_fits = M <= kSkinnyMaxRows && words;
  GB_REQUIRE(which != 2 || skinny_fits, "gemm_f32: the skinny kernel takes at most %d rows of 16-byte words (M=%d K=%d)",
             kSkinnyMaxRows, M, K);
  if (which == 2 || (which == 0 && skinny_fits)) {
    if (M <= 1) launch_skinny<1>(a, lda, w, ldw, c, ldc, M, N, K, accumulate, stream);
    else if (M <= 2) launch_skinny<2>(a, lda, w, ldw, c, ldc, M, N, K, accumulate, stream);
    else if (M <= 4) launch_skinny<4>(a, lda, w, ldw, c, ldc, M, N, K, accumulate, stream);
    else if (M <= 8) launch_skinny<8>(a, lda, w, ldw, c, ldc, M, N, K, accumulate, stream);
    else launch_skinny<16>(a, lda, w, ldw, c, ldc, M, N, K, accumulate, stream);
    return launched("gemm_f32 (skinny)");
  }
  GB_REQUIRE(which != 3 || words, "gemm_f32: the wide kernel takes rows of 16-byte words (K=%d lda=%d ldw=%d)", K, lda, ldw);
  const dim3 wide((N + WN - 1) / WN, (M + WM - 1) / WM);
  if (which == 3 || (which == 0 && words && (long long)wide.x * wide.y >= kWideMinTiles)) {
    GB_REQUIRE(wide.y <= 65535, "gemm_f32: M=%d needs more than 65535 row tiles", M);
    hipLaunchKernelGGL(gemm_f32_wide_kernel, wide, dim3(256), 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
    return launched("gemm_f32 (wide)");
  }
  const dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  GB_REQUIRE(grid.y <= 65535, "gemm_f32: M=%d needs more than 65535 row tiles", M);
  hipLaunchKernelGGL(gemm_f32_kernel, grid, dim3(256), 0, stream, a, lda, w, ldw, c, ldc, M, N, K, accumulate);
  return launched("gemm_f32");
}

extern "C" int gb_gemm_f32(const float* a, int lda, const float* w, int ldw, float* c, int ldc, int M, int N, int K,
                           int accumulate, hipStream_t stream) {
  return gb_gemm_f32_by(a, lda, w, ldw, c, ldc, M, N, K, accumulate, 0, stream);
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_gemm_f32)
GB_TAPED(gb_gemm_f32_by)
