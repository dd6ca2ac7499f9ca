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
// grid (row tiles of W).  A workgroup of WAVES waves owns 16 rows of W and walks all of k in slices
// of ITERS*WAVES*64: wave w takes the 64-wide k blocks w, w+WAVES, ... of a slice; inside a block
// lane group q holds k = 16q..16q+15 as two operands of 8 (the same split for W and for A, so the
// products pair up).  All loads of a slice are issued before its first MFMA.  The waves combine
// through LDS in wave order.  Few rows of W (a small N) are given many waves each, so that the
// launch still keeps enough loads in flight to use the memory system; no partial result ever
// leaves the workgroup, so no pass over memory is needed to combine them.
//
// EPI_STORE / EPI_ACCUMULATE: C[m, n] = or += the product.  EPI_SILU_MUL: W holds gate rows
// [0, N/2) and up rows [N/2, N); a tile takes 8 gate rows and the 8 up rows that belong to them
// and writes act[m, j] = gate / (1 + exp(-gate)) * up (crates/glassbox-core/src/model.rs:336-340)
// to C[M, N/2].
enum : int { EPI_STORE = 0, EPI_ACCUMULATE = 1, EPI_SILU_MUL = 2 };

template <int MT, int WAVES, int ITERS, int RT, int EPI, typename CT>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16* __restrict__ a, int lda,
                                                                 const bf16* __restrict__ w, int ldw, CT* __restrict__ c,
                                                                 int ldc, int M, int N, int K) {
  __shared__ float part[WAVES][RT][MT][64][4];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const bf16* wrow[RT];
  bool row_ok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int tile = blockIdx.x * RT + rt;
    int row;
    if (EPI == EPI_SILU_MUL) row = r < 8 ? tile * 8 + r : N / 2 + tile * 8 + (r - 8);
    else row = tile * 16 + r;
    row_ok[rt] = EPI == EPI_SILU_MUL ? (tile * 8 + (r & 7) < N / 2) : row < N;
    wrow[rt] = w + (size_t)(row_ok[rt] ? row : 0) * ldw;
  }

  f32x4 acc[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[rt][t][e] = 0.f;

  // a 64-wide k block is two MFMA steps of 32: lane group q holds k = 8q..8q+7 of each
  for (int kbeg = 0; kbeg < K; kbeg += ITERS * WAVES * 64) {
    bf16x8 wf[RT][ITERS][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int k = kbeg + (wave + WAVES * it) * 64 + q * 8;
        wf[rt][it][0] = (row_ok[rt] && k < K) ? load8(wrow[rt] + k) : zero8();
        wf[rt][it][1] = (row_ok[rt] && k + 32 < K) ? load8(wrow[rt] + k + 32) : zero8();
      }
    if (MT == 1) {
      const bf16* arow = a + (size_t)(r < M ? r : 0) * lda;
      bf16x8 xf[ITERS][2];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int k = kbeg + (wave + WAVES * it) * 64 + q * 8;
        xf[it][0] = (r < M && k < K) ? load8(arow + k) : zero8();
        xf[it][1] = (r < M && k + 32 < K) ? load8(arow + k + 32) : zero8();
      }
#pragma unroll
      for (int it = 0; it < ITERS; ++it)
#pragma unroll
        for (int rt = 0; rt < RT; ++rt) {
          acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][0], xf[it][0], acc[rt][0], 0, 0, 0);
          acc[rt][0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][1], xf[it][1], acc[rt][0], 0, 0, 0);
        }
    } else {
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int k = kbeg + (wave + WAVES * it) * 64 + q * 8;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const int m = t * 16 + r;
          const bf16* arow = a + (size_t)(m < M ? m : 0) * lda;
          const bf16x8 x0 = (m < M && k < K) ? load8(arow + k) : zero8();
          const bf16x8 x1 = (m < M && k + 32 < K) ? load8(arow + k + 32) : zero8();
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][0], x0, acc[rt][t], 0, 0, 0);
            acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][1], x1, acc[rt][t], 0, 0, 0);
          }
        }
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) part[wave][rt][t][lane][e] = acc[rt][t][e];
  __syncthreads();
  if (tid >= 256) return;

  // D[n, m]: lane l holds column m = l%16 and rows n = 4*(l/16) + e.  The first 256 threads own the
  // cells of the tiles: thread tid owns cell (l = tid/4, e = tid%4) of every row tile and column block.
  const int l = tid / 4, e = tid % 4;
  float v[RT][MT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      float s = part[0][rt][t][l][e];
#pragma unroll
      for (int wv = 1; wv < WAVES; ++wv) s += part[wv][rt][t][l][e];
      v[rt][t] = s;
    }
  const int nrow = 4 * (l / 16) + e;  // row of the tile, 0..15
  if (EPI == EPI_SILU_MUL) {
    // rows 0..7 are gate, 8..15 the matching up rows: the up values travel through LDS.  Only the
    // first four waves are here; the slice of the last wave is free once every sum above is done.
    float* up = &part[WAVES - 1][0][0][0][0];
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int t = 0; t < MT; ++t) up[(rt * MT + t) * 256 + tid] = v[rt][t];
    __syncthreads();
    if (nrow < 8) {
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        const int j = (blockIdx.x * RT + rt) * 8 + nrow;
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          const int m = t * 16 + l % 16;
          const float g = v[rt][t], u = up[(rt * MT + t) * 256 + tid + 128];
          if (m < M && j < N / 2) c[(size_t)m * ldc + j] = (CT)(g / (1.0f + __expf(-g)) * u);
        }
      }
    }
  } else {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n = (blockIdx.x * RT + rt) * 16 + nrow;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + l % 16;
        if (m < M && n < N) store_c<CT>(c + (size_t)m * ldc + n, v[rt][t], EPI == EPI_ACCUMULATE);
      }
    }
  }
}

// Waves per workgroup, loads in flight per wave and row tiles per workgroup.
// GB_SKINNY="waves,iters,rowtiles" overrides (for measurements).
inline void skinny_plan(int tiles, int K, int mt, int* waves, int* iters, int* rt) {
  // measured on SmolLM2-1.7B and Llama-3-8B shapes: sixteen waves a workgroup keep the most loads in
  // flight; two row tiles a workgroup halve the re-reading of A once there are tiles enough
  const int blocks = (K + 63) / 64;               // 64-wide k blocks
  *waves = blocks >= 16 ? 16 : 4;
  *rt = tiles >= 256 ? 2 : 1;
  const int per_wave = (blocks + *waves - 1) / *waves;
  *iters = (mt == 1 && per_wave >= 2) ? 2 : 1;
  if (const char* env = getenv("GB_SKINNY")) {
    int wv = 0, it = 0, r = 0;
    if (sscanf(env, "%d,%d,%d", &wv, &it, &r) == 3 && (wv == 4 || wv == 16) && (it == 1 || (it == 2 && mt == 1)) &&
        (r == 1 || r == 2)) {
      *waves = wv;
      *iters = it;
      *rt = r;
    }
  }
}

template <int MT, int EPI, typename CT>
int launch_skinny_mt(int tiles, const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K,
                     hipStream_t stream) {
  int waves, iters, rt;
  skinny_plan(tiles, K, MT, &waves, &iters, &rt);
#define GB_CFG(WV, IT, RT)                                                                                                \
  if (waves == WV && iters == (IT) && rt == RT)                                                                           \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, WV, (IT), RT, EPI, CT>), dim3((tiles + RT - 1) / RT), dim3(WV * 64), 0, stream, \
                       a, lda, w, ldw, c, ldc, M, N, K);
  // the configurations skinny_plan can ask for: two loads in flight only with one column block
  GB_CFG(4, 1, 1) GB_CFG(4, 1, 2) GB_CFG(16, 1, 1) GB_CFG(16, 1, 2)
  if (MT == 1) {
    GB_CFG(4, MT == 1 ? 2 : 1, 1) GB_CFG(4, MT == 1 ? 2 : 1, 2) GB_CFG(16, MT == 1 ? 2 : 1, 1) GB_CFG(16, MT == 1 ? 2 : 1, 2)
  }
#undef GB_CFG
  return launched("gemm_bf16 (skinny)");
}

template <int EPI, typename CT>
int launch_skinny(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, hipStream_t stream) {
  const int tiles = EPI == EPI_SILU_MUL ? (N / 2 + 7) / 8 : (N + 15) / 16;
  const int mt = (M + 15) / 16;
  if (mt == 1) return launch_skinny_mt<1, EPI, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, stream);
  if (mt == 2) return launch_skinny_mt<2, EPI, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, stream);
  if (mt == 3) return launch_skinny_mt<3, EPI, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, stream);
  return launch_skinny_mt<4, EPI, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, stream);
}

}  // namespace

// epilogue: 0 store, 1 accumulate (float32 C), 2 SiLU-multiply of stacked gate/up rows (C is [M, N/2]).
extern "C" int gb_gemm_bf16(const void* a, int lda, const void* w, int ldw, void* c, int ldc, int c_dtype, int M, int N,
                            int K, int epilogue, hipStream_t stream) {
  GB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  GB_REQUIRE(K % 8 == 0, "gemm_bf16: the inner size K=%d must be a multiple of 8 (16-byte operand loads)", K);
  GB_REQUIRE(lda % 8 == 0 && ldw % 8 == 0, "gemm_bf16: row strides (%d, %d) must be multiples of 8 elements", lda, ldw);
  GB_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm_bf16: unknown epilogue %d", epilogue);
  const int ncols = epilogue == EPI_SILU_MUL ? N / 2 : N;
  GB_REQUIRE(epilogue != EPI_SILU_MUL || N % 2 == 0, "gemm_bf16: stacked gate/up rows need an even N, got %d", N);
  GB_REQUIRE(lda >= K && ldw >= K && ldc >= ncols, "gemm_bf16: a leading dimension is shorter than its row");
  GB_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  GB_REQUIRE(epilogue != EPI_ACCUMULATE || c_dtype == kF32, "gemm_bf16: accumulation is into a float32 result");
  GB_REQUIRE(epilogue != EPI_SILU_MUL || M <= 64, "gemm_bf16: the fused SiLU-multiply serves up to 64 rows, got %d", M);
  GB_REQUIRE(c_dtype == kF32 || c_dtype == kBF16, "gemm_bf16: unknown result dtype %d", c_dtype);
  if (M == 0) return 0;
  const bf16* A = (const bf16*)a;
  const bf16* W = (const bf16*)w;
  if (M <= 64) {
#define GB_SK(EPI, CT) return launch_skinny<EPI, CT>(A, lda, W, ldw, (CT*)c, ldc, M, N, K, stream)
    if (epilogue == EPI_STORE && c_dtype == kF32) GB_SK(EPI_STORE, float);
    if (epilogue == EPI_STORE && c_dtype == kBF16) GB_SK(EPI_STORE, bf16);
    if (epilogue == EPI_ACCUMULATE) GB_SK(EPI_ACCUMULATE, float);
    if (epilogue == EPI_SILU_MUL && c_dtype == kF32) GB_SK(EPI_SILU_MUL, float);
    GB_SK(EPI_SILU_MUL, bf16);
#undef GB_SK
  }
  const dim3 grid((N + TBN - 1) / TBN, (M + TBM - 1) / TBM), block(256);
  GB_REQUIRE(grid.y <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  if (c_dtype == kF32)
    hipLaunchKernelGGL(gemm_tiled_kernel<float>, grid, block, 0, stream, A, lda, W, ldw, (float*)c, ldc, M, N, K,
                       epilogue == EPI_ACCUMULATE);
  else
    hipLaunchKernelGGL(gemm_tiled_kernel<bf16>, grid, block, 0, stream, A, lda, W, ldw, (bf16*)c, ldc, M, N, K, 0);
  return launched("gemm_bf16 (tiled)");
}
