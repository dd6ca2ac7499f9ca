// bfloat16 matrix products on the matrix cores (MFMA), 32-bit accumulation:
//   C[M,N] (+)= A[M,K] . W[N,K]^T,   W in the nn.Linear layout [out, in]
// (crates/glassbox-core/src/kernels.rs:381,586).  Both operands are contiguous along k, which
// is the layout MFMA operands want: every lane loads 8 consecutive k as one 16-byte word.
//
// Five kernels:
//  * tiled  (M > 64, prompt portions): a workgroup of 2x2 waves, each wave a block of 2x2 or 2x1
//    v_mfma_f32_32x32x16_bf16 tiles (workgroup tile 128x128 or 128x64; 64 rows high where the taller tiles would be
//    few), operands staged through LDS in k-steps of 64 with two buffers; the SiLU-multiply of stacked gate/up rows
//    can be its epilogue.  Its workgroups can also divide k (split k: a second pass adds their sums in order).
//  * stream (65 to 128 rows, the mixed steps of serving): 128 x 32 or 128 x 64 tiles, both operands through deep
//    rings in LDS, W asked for by a wave of its own.
//  * ring   (a thousand rows and more, enough 256x256 tiles to fill the chip): 2x4 waves, a wave 4x2 such
//    tiles; operands go from memory straight into a ring of LDS buffers in k-steps of 32.
//  * skinny (M <= 64, decoding): bound by reading W once.  A workgroup owns 16 or 32 rows of W (8 where the
//    rows of W are few); its
//    waves take interleaved 64-wide k blocks, stream W straight from memory into MFMA operands
//    (v_mfma_f32_16x16x32_bf16, W as the A operand so that the 16 rows fill the tile) and combine
//    through LDS in a fixed order; it can norm float32 rows on the way, apply the SiLU-multiply, or
//    (the QKV product) rotate the heads and write the key/value cache, or prepare the next norm where it adds
//    into the residual.
//  * folded (M <= 8 and few rows of W): the skinny kernel with two k ranges side by side in a tile,
//    so that a workgroup owns 8 rows of W and there are twice as many workgroups.
// In all, every output cell is summed in an order fixed by (K, kernel) alone, not by M or by
// the cell's neighbours.  C is bfloat16 or float32; accumulation (+=) is into float32.
#include <type_traits>

#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
// read once and not again in this kernel: the caches need not keep it
__device__ __forceinline__ bf16x8 load8_once(const bf16* p) { return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p)); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

// What a product of at most 64 rows may do for the RMS norm that follows it or precedes it.
//  * emit (the folded kernel for up to 8 rows, the skinny kernel beyond; accumulating into the float32 residual):
//    besides the new residual r it writes h[m, n] = bf16(gamma[n] * r[m, n]), the operand of the next product, and
//    for every tile of columns (8 or 16: gb_gemm_bf16_emit_parts says how many tiles) the sums over them of
//    r[m, n]^2 to ss[tile * stride + m]: the next norm's pass over the residual is done where the residual is made.
//    stride = parts_stride(M): 8 for up to 8 rows, 64 beyond.
//  * parts (the skinny kernel): the rows of A are such an h; the product is scaled by
//    1 / sqrt(sum of the n_parts partial sums of row m / K + eps), added up in the order of the tiles.
__host__ __device__ __forceinline__ int parts_stride(int M) { return M <= 8 ? 8 : 64; }
struct NormExtras {
  const void* emit_gamma;
  int emit_gamma_f32;
  bf16* emit_h;
  int emit_ldh;
  float* emit_ss;
  const float* parts;
  int n_parts;
};

// EPI_ROPE (the skinny kernel; the QKV product of a decode step): W stacks nh query heads, nkv key heads
// and nkv value heads of hd rows each.  The product rotates query and key heads by the angles of each
// row's position (pairs (i, i + hd/2), crates/glassbox-core/src/model.rs:102-115) while the sums are
// still 32-bit, writes the stacked rows to C as usual, and the key and value heads straight into the
// cache pages at slots[m] (keys [page][kv head][hd / 8][slot][8], values [page][kv head][hd][slot]) if slots is
// given: the rotation kernel and its round trip through memory are not needed.
struct RopeExtras {
  const float* cosv;   // [M][hd/2], nullptr: no rotation
  const float* sinv;
  const int32_t* slots;  // [M], nullptr: nothing is stored
  bf16* k_pages;
  bf16* v_pages;
  int nh, nkv, hd, page_size;
  int three_halves;  // the launch gives a workgroup a tile and a half (see three_halves_tile), not two tiles
};

// Tiles of the skinny kernel's rotating product, 8 pairs each, dealt a tile and a half to a workgroup: workgroup g
// takes tile 3g/2 whole and the first four pairs of the next (g even), or the last four pairs of tile (3g - 1)/2 and
// the next whole (g odd).  384 tiles (the 6,144 rows of a QKV product) then make 256 workgroups of equal work, one for
// every compute unit, where two tiles each would make 192.  [lo, hi): the pairs of tile rt that are the workgroup's.
__device__ __forceinline__ int three_halves_tile(int g, int rt, int* lo, int* hi) {
  *lo = (g & 1) && rt == 0 ? 4 : 0;
  *hi = !(g & 1) && rt == 1 ? 4 : 8;
  return ((g & 1) ? (3 * g - 1) / 2 : 3 * g / 2) + rt;
}

template <typename CT> __device__ __forceinline__ void store_c(CT* c, float v, int accumulate);
template <> __device__ __forceinline__ void store_c<float>(float* c, float v, int accumulate) { *c = accumulate ? *c + v : v; }
template <> __device__ __forceinline__ void store_c<bf16>(bf16* c, float v, int) { *c = (bf16)v; }

// ------------------------------------------------------------------------- tiled
// A workgroup of 2 x 2 waves; a wave owns WM x WN tiles of 32 x 32, so the workgroup's tile is
// (64 WM) x (64 WN).  Operands are staged through LDS in k-steps of 64, two buffers; rows are padded
// to 144 bytes so that the 16-byte operand reads of a wave spread over the banks.
//
// EPI_SILU_MUL (WN = 2): W stacks gate rows [0, N/2) over up rows [N/2, N).  Of a wave's two column
// tiles the first holds 32 gate columns and the second the 32 up columns that belong to them, so
// act = gate / (1 + exp(-gate)) * up (crates/glassbox-core/src/model.rs:336-340) is formed in
// registers and C is [M, N/2].
enum : int { EPI_STORE = 0, EPI_ACCUMULATE = 1, EPI_SILU_MUL = 2, EPI_ROPE = 3 };
constexpr int TBK = 64, TLD = TBK + 8;  // k-step; LDS row stride in elements (144 bytes)
constexpr int TCPR = TBK / 8;           // 16-byte chunks per row of a k-step
constexpr int TKS = TBK / 16;           // MFMA k-steps per LDS k-step

template <int WM, int WN, int DEPTH, int EPI, bool KFULL, typename CT>
__global__ __launch_bounds__(256, WN == 2 ? 2 : 1) void gemm_tiled_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w,
                                                         int ldw, CT* __restrict__ c, int ldc, int M, int N, int K,
                                                         int k_slice) {
  constexpr int BM = 64 * WM, BN = 64 * WN;
  constexpr int CA = BM * TCPR / 256, CW = BN * TCPR / 256;  // chunks a thread moves per k-step
  if (k_slice > 0) {  // split k: workgroup z of a tile sums its own slice of k into its own copy of C
    const int z = blockIdx.z;
    a += (size_t)z * k_slice;
    w += (size_t)z * k_slice;
    c += (size_t)z * M * ldc;
    K = min(k_slice, K - z * k_slice);
  }
  __shared__ __attribute__((aligned(16))) bf16 As[2][BM][TLD];
  __shared__ __attribute__((aligned(16))) bf16 Ws[2][BN][TLD];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / 2, wn = wave % 2;
  const int m0 = blockIdx.y * BM;
  const int half = N / 2;  // EPI_SILU_MUL: number of gate rows
  // row of W behind row r of the workgroup's W tile (r = wn*32*WN + j*32 + column)
  auto w_row = [&](int r) -> int {
    if (EPI == EPI_SILU_MUL) {
      const int wv = r / 64, j = (r % 64) / 32, col = r % 32;
      const int n = blockIdx.x * 64 + wv * 32 + col;
      return n < half ? (j ? half + n : n) : -1;
    }
    const int n = blockIdx.x * BN + r;
    return n < N ? n : -1;
  };

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // Chunks on their way from memory to LDS wait in registers, DEPTH k-steps' worth: a load has DEPTH
  // k-steps of arithmetic to arrive in before its registers are written to LDS.  Within a k-step the
  // LDS writes and the loads that refill their registers are spread over the first three of the four
  // MFMA steps, so that memory requests and arithmetic are issued side by side, not in bursts.
  // Rows beyond M or N are read from a row that exists (their results are never stored), so that the
  // loop has no branch around a load.
  constexpr int CT_ = CA + CW;
  bf16x8 held[DEPTH][CT_];
  const bf16* src[CT_];
#pragma unroll
  for (int ci = 0; ci < CT_; ++ci) {
    const int ch = tid + 256 * (ci < CA ? ci : ci - CA);
    if (ci < CA) {
      src[ci] = a + (size_t)min(m0 + ch / TCPR, M - 1) * lda + (ch % TCPR) * 8;
    } else {
      src[ci] = w + (size_t)max(w_row(ch / TCPR), 0) * ldw + (ch % TCPR) * 8;
    }
  }
  auto fetch = [&](int ci, int k0, auto set) {
    if constexpr (KFULL) {
      held[decltype(set)::value][ci] = load8(src[ci] + k0);
    } else {
      const int ch = tid + 256 * (ci < CA ? ci : ci - CA);
      held[decltype(set)::value][ci] = k0 + (ch % TCPR) * 8 < K ? load8(src[ci] + k0) : zero8();
    }
  };
  auto stash = [&](int ci, int buf, auto set) {
    const int ch = tid + 256 * (ci < CA ? ci : ci - CA);
    bf16* dst = ci < CA ? &As[buf][ch / TCPR][(ch % TCPR) * 8] : &Ws[buf][ch / TCPR][(ch % TCPR) * 8];
    *reinterpret_cast<bf16x8*>(dst) = held[decltype(set)::value][ci];
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;
  using Yes = std::true_type;
  using No = std::false_type;

  const int steps = (K + TBK - 1) / TBK;
  const int arow = wm * 32 * WM + lane % 32, wrow = wn * 32 * WN + lane % 32, koff = 8 * (lane / 32);
  bf16x8 fa[2][WM], fw[2][WN];  // operands of MFMA step ks+1 are read from LDS while the MFMAs of step ks run
  auto read_operands = [&](int buf, int kk, int into) {
#pragma unroll
    for (int i = 0; i < WM; ++i) fa[into][i] = *reinterpret_cast<const bf16x8*>(&As[buf][arow + i * 32][kk * 16 + koff]);
#pragma unroll
    for (int j = 0; j < WN; ++j) fw[into][j] = *reinterpret_cast<const bf16x8*>(&Ws[buf][wrow + j * 32][kk * 16 + koff]);
  };
  // k-step s is computed from LDS buffer s % 2.  Register set `other` holds k-step s + 1: it is written
  // to the other buffer (if there is a k-step s + 1: more), and loaded again with k-step s + 1 + DEPTH
  // (if there is one: refill).  The barrier stands before the last MFMA step: by then every wave has
  // written its part of k-step s + 1 and has read the last operands of k-step s, so the last MFMA
  // step can already read the first operands of k-step s + 1.
  static_assert(TKS == 4, "the schedule below is written for four MFMA steps per k-step");
  auto step = [&](int s, auto other, auto more, auto refill) {
    const int buf = s & 1;
#pragma unroll
    for (int ks = 0; ks < TKS; ++ks) {
      const int cur = ks & 1, nxt = cur ^ 1;
      if (ks + 1 < TKS)
        read_operands(buf, ks + 1, nxt);
      else if (decltype(more)::value)
        read_operands(buf ^ 1, 0, nxt);
      if (ks < 3) {
#pragma unroll
        for (int ci = ks; ci < CT_; ci += 3) {
          if (decltype(more)::value) stash(ci, buf ^ 1, other);
          if (decltype(refill)::value) fetch(ci, (s + 1 + DEPTH) * TBK, other);
        }
      }
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[cur][i], fw[cur][j], acc[i][j], 0, 0, 0);
      if (ks == 2) __syncthreads();
      __builtin_amdgcn_sched_barrier(0);  // each MFMA step keeps its share of the memory traffic
    }
  };

  auto any_step = [&](int s, auto other) {  // near the end fewer and fewer k-steps have something ahead of them
    if (s + 1 + DEPTH < steps)
      step(s, other, Yes{}, Yes{});
    else if (s + 1 < steps)
      step(s, other, Yes{}, No{});
    else
      step(s, other, No{}, No{});
  };
#pragma unroll
  for (int ci = 0; ci < CT_; ++ci) fetch(ci, 0, Set0{});
  if (DEPTH == 2 && steps > 1) {
#pragma unroll
    for (int ci = 0; ci < CT_; ++ci) fetch(ci, TBK, std::integral_constant<int, DEPTH - 1>{});
  }
#pragma unroll
  for (int ci = 0; ci < CT_; ++ci) stash(ci, 0, Set0{});
  if (steps > DEPTH) {
#pragma unroll
    for (int ci = 0; ci < CT_; ++ci) fetch(ci, DEPTH * TBK, Set0{});
  }
  __syncthreads();
  read_operands(0, 0, 0);
  int s = 0;
  if constexpr (DEPTH == 2) {
    for (; s + 4 < steps; s += 2) {  // both k-steps of a round have a k-step three ahead
      step(s, Set1{}, Yes{}, Yes{});
      step(s + 1, Set0{}, Yes{}, Yes{});
    }
    for (; s < steps; s += 2) {
      any_step(s, Set1{});
      if (s + 1 < steps) any_step(s + 1, Set0{});
    }
  } else {
    for (; s + 2 < steps; ++s) step(s, Set0{}, Yes{}, Yes{});
    for (; s < steps; ++s) any_step(s, Set0{});
  }

  // accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
  if (EPI == EPI_SILU_MUL) {
    const int gn = blockIdx.x * 64 + wn * 32 + lane % 32;
    if (gn >= half) return;
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm * 32 * WM + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        const float g = acc[i][0][r], u = acc[i][WN - 1][r];
        if (gm < M) c[(size_t)gm * ldc + gn] = (CT)(g / (1.0f + __expf(-g)) * u);
      }
    return;
  }
  if constexpr (EPI == EPI_ACCUMULATE) {
    // a wave whose tiles lie wholly inside C reads all old values of a tile before it adds: behind the checks
    // below every read would wait for the one before it
    if (m0 + (wm + 1) * 32 * WM <= M && blockIdx.x * BN + (wn + 1) * 32 * WN <= N) {
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          CT* base = c + (size_t)(m0 + wm * 32 * WM + i * 32 + 4 * (lane / 32)) * ldc + blockIdx.x * BN + wn * 32 * WN + j * 32 + lane % 32;
          float old[16];
#pragma unroll
          for (int r = 0; r < 16; ++r) old[r] = (float)base[(size_t)(8 * (r / 4) + r % 4) * ldc];
#pragma unroll
          for (int r = 0; r < 16; ++r) base[(size_t)(8 * (r / 4) + r % 4) * ldc] = (CT)(old[r] + acc[i][j][r]);
        }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j) {
      const int gn = blockIdx.x * BN + wn * 32 * WN + j * 32 + lane % 32;
      if (gn >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm * 32 * WM + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (gm < M) store_c<CT>(c + (size_t)gm * ldc + gn, acc[i][j][r], EPI == EPI_ACCUMULATE);
      }
    }
}

// Tile of the workgroup, 128 x (64 WN), and the depth of the register prefetch.  128 x 128 re-reads
// the operands least; 128 x 64 when that would leave compute units idle.  The wide tile's registers
// allow two workgroups a compute unit only with one k-step of prefetch, the narrow tile's with two.
inline void tiled_plan(int M, int N, int* wn, int* depth) {
  const int blocks = ((M + 127) / 128) * ((N + 127) / 128);
  *wn = blocks < 384 ? 1 : 2;
  *depth = *wn == 1 ? 2 : 1;
}

template <int EPI, typename CT>
int launch_tiled(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, hipStream_t stream) {
  int wn, depth;
  tiled_plan(M, N, &wn, &depth);
  if (EPI == EPI_SILU_MUL) wn = 2;  // a wave's two column tiles are gate and up
  const int cols = EPI == EPI_SILU_MUL ? N / 2 : N, bn = EPI == EPI_SILU_MUL ? 64 : 64 * wn;
  // Tiles of 64 rows where those of 128 would leave a third of the compute units without a workgroup (the
  // products of a narrow model at some hundred rows): a workgroup's time is its k-steps' arithmetic, and half the
  // rows halve it.  A SiLU-multiply product, whose workgroups take 128 rows of W each, gains up to 300 workgroups
  // (two of the smaller ones share a compute unit: gate/up of 256 rows on SmolLM2-1.7B shapes 34 -> 30 us, of 640 to
  // 896 rows on SmolLM2-360M shapes 17 -> 14 and 24 -> 20 us; the other products lose from 168 on).
  const bool low = M > 64 && ((cols + bn - 1) / bn) * ((M + 127) / 128) < (EPI == EPI_SILU_MUL ? 300 : 168);
  const int bm = low ? 64 : 128;
  const dim3 grid((cols + bn - 1) / bn, (M + bm - 1) / bm), block(256);
  GB_REQUIRE(grid.y <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  const bool kfull = K % TBK == 0;  // then no load needs a check against K
#define GB_T(WM, B, D)                                                                                                      \
  if (wn == (B) && depth == (D)) {                                                                                          \
    if (kfull)                                                                                                              \
      hipLaunchKernelGGL((gemm_tiled_kernel<WM, (B), (D), EPI, true, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, \
                         N, K, 0);                                                                                          \
    else                                                                                                                    \
      hipLaunchKernelGGL((gemm_tiled_kernel<WM, (B), (D), EPI, false, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc,  \
                         M, N, K, 0);                                                                                       \
  }
  if (low) {
    depth = wn == 1 ? 2 : 1;
    GB_T(1, 2, 1)
    if (EPI != EPI_SILU_MUL) { GB_T(1, (EPI == EPI_SILU_MUL ? 2 : 1), 2) }
  } else {
    GB_T(2, 2, 1) GB_T(2, 2, 2)
    if (EPI != EPI_SILU_MUL) { GB_T(2, (EPI == EPI_SILU_MUL ? 2 : 1), 1) GB_T(2, (EPI == EPI_SILU_MUL ? 2 : 1), 2) }
  }
#undef GB_T
  return launched("gemm_bf16 (tiled)");
}

// ------------------------------------------------------------------------- ring
// Large products (many rows, many 256 x 256 tiles): a workgroup of 2 x 4 waves with a 256 x 256 tile, a wave
// 4 x 2 tiles of 32 x 32.  The larger tile halves the operand bytes a flop needs, which is what bounds the
// 128-wide kernel.  Operands go from memory straight into LDS (global_load_lds, 16 bytes a lane: a wave's
// instruction fills 1 KB of LDS in lane order, so the lane decides which piece of memory lands where), in
// k-steps of 32 through a ring of RING_STAGES buffers: nothing waits in registers, and a load has
// RING_STAGES - 1 k-steps to arrive in.  A row of a k-step is 64 bytes = 4 pieces; piece c of row r lies at
// position c ^ ((r >> 2) & 3), which spreads the 16-byte operand reads of a wave over all banks.
//
// The compiler knows nothing of what those loads write: before every LDS read it would wait for all of them.
// So the operand reads are inline assembly, and the waits are written here by hand:
//   * lgkmcnt before the MFMAs that use an operand;
//   * the barrier of k-step s stands between its two MFMA steps.  Before it a wave waits for its last operand
//     reads of stage s (lgkmcnt) and for its own loads of stage s + 1 (vmcnt: loads retire in order).  After
//     it, every wave's loads of stage s + 1 have landed, so its operands may be read (they arrive under the
//     second MFMA step), and every wave is done with stage s, so the loads of k-step s + 1 may overwrite it.
constexpr int RBK = 32, RING_STAGES = 4;
constexpr int RGM = 2, RGN = 4, RTM = 4, RTN = 2;          // waves along m, n; 32 x 32 tiles of a wave along m, n
constexpr int RBM = RGM * RTM * 32, RBN = RGN * RTN * 32;  // 256 x 256
constexpr int RLA = RBM / 16 / (RGM * RGN), RLW = RBN / 16 / (RGM * RGN), RLPS = RLA + RLW;  // loads of a wave per stage
typedef __attribute__((address_space(3))) void lds_void;
typedef __attribute__((address_space(1))) const void glb_void;

__device__ __forceinline__ bf16x8 lds_read16(uint32_t addr) {
  bf16x8 v;
  asm volatile("ds_read_b128 %0, %1" : "=v"(v) : "v"(addr) : "memory");
  return v;
}
// waits until at most LEFT LDS reads are outstanding; the operands named become usable
template <int LEFT, int NA, int NB>
__device__ __forceinline__ void lds_wait(bf16x8 (&fa)[NA], bf16x8 (&fb)[NB]) {
  asm volatile("s_waitcnt lgkmcnt(%0)" ::"n"(LEFT) : "memory");
#pragma unroll
  for (int i = 0; i < NA; ++i) asm volatile("" : "+v"(fa[i]));
#pragma unroll
  for (int j = 0; j < NB; ++j) asm volatile("" : "+v"(fb[j]));
}
// waits until at most LEFT of this wave's loads from memory are on their way (the counter's six bits lie in two
// places of the instruction's operand: bits 3:0 and 15:14; the other counters are left alone)
template <int LEFT> __device__ __forceinline__ void vm_wait() {
  static_assert(LEFT >= 0 && LEFT < 64, "the counter has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (LEFT & 15) | ((LEFT >> 4) << 14));
}

template <int EPI, typename CT>
__global__ __launch_bounds__(RGM * RGN * 64, 1) void gemm_ring_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w, int ldw,
                                                           CT* __restrict__ c, int ldc, int M, int N, int K, int k_slice) {
  int bx = blockIdx.x, by = blockIdx.y;
  if (k_slice > 0) {  // split k: workgroup z of a tile sums its own slice of k into its own copy of C
    int z = blockIdx.z;
    // The chip deals workgroups round its 8 dies by their number, and each die has a second-level cache of its
    // own.  With the grid as it stands a die would hold one column tile over all row tiles and all slices (8 + 32
    // different operand pieces a k-step among its 32 workgroups); numbered anew, it holds an eighth of the grid in
    // a row: one slice, some row tiles, all column tiles (4 + 8 pieces), which its cache then serves.
    const int gx = gridDim.x, gy = gridDim.y, total = gx * gy * gridDim.z;
    if (total % 8 == 0) {
      const int id = bx + gx * (by + gy * z), anew = (id % 8) * (total / 8) + id / 8;
      bx = anew % gx;
      by = (anew / gx) % gy;
      z = anew / (gx * gy);
    }
    a += (size_t)z * k_slice;
    w += (size_t)z * k_slice;
    c += (size_t)z * M * ldc;
    K = min(k_slice, K - z * k_slice);
  }
  __shared__ __attribute__((aligned(16))) bf16 As[RING_STAGES][RBM * RBK];
  __shared__ __attribute__((aligned(16))) bf16 Ws[RING_STAGES][RBN * RBK];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int wm = wave / RGN, wn = wave % RGN;
  const int m0 = by * RBM;
  const int half = N / 2;  // EPI_SILU_MUL: number of gate rows
  // row of W behind row r of the workgroup's W tile (r = wn * 64 + j * 32 + column); with EPI_SILU_MUL a wave's
  // first column tile holds gate rows and its second the up rows that belong to them
  auto w_row = [&](int r) -> int {
    if (EPI == EPI_SILU_MUL) {
      const int j = (r % (RTN * 32)) / 32;  // column tile of its wave: even ones hold gate rows, odd ones their up rows
      const int n = bx * (RBN / 2) + (r / (RTN * 32)) * (RTN / 2 * 32) + (j / 2) * 32 + r % 32;
      return n < half ? (j % 2 ? half + n : n) : 0;
    }
    return min(bx * RBN + r, N - 1);
  };
  // a wave's load instruction moves 16 rows x 4 pieces; rows beyond M or N are read from a row that exists
  const bf16* asrc[RLA];
  const bf16* wsrc[RLW];
#pragma unroll
  for (int t = 0; t < RLA; ++t) {
    const int row = (wave * RLA + t) * 16 + lane / 4, piece = (lane % 4) ^ ((row >> 2) & 3);
    asrc[t] = a + (size_t)min(m0 + row, M - 1) * lda + piece * 8;
  }
#pragma unroll
  for (int t = 0; t < RLW; ++t) {
    const int row = (wave * RLW + t) * 16 + lane / 4, piece = (lane % 4) ^ ((row >> 2) & 3);
    wsrc[t] = w + (size_t)w_row(row) * ldw + piece * 8;
  }
  auto load_a = [&](int t, int stage, int k0) {
    __builtin_amdgcn_global_load_lds((glb_void*)(asrc[t] + k0), (lds_void*)&As[stage][(wave * RLA + t) * 16 * RBK], 16, 0, 0);
  };
  auto load_w = [&](int t, int stage, int k0) {
    __builtin_amdgcn_global_load_lds((glb_void*)(wsrc[t] + k0), (lds_void*)&Ws[stage][(wave * RLW + t) * 16 * RBK], 16, 0, 0);
  };
  f32x16 acc[RTM][RTN];
#pragma unroll
  for (int i = 0; i < RTM; ++i)
#pragma unroll
    for (int j = 0; j < RTN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  // operand of MFMA step ks (0, 1): row lane % 32 of a 32-row tile, piece 2 ks + lane / 32
  uint32_t off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) off[ks] = 2 * ((lane % 32) * RBK + (((2 * ks + lane / 32) ^ ((lane >> 2) & 3)) * 8));
  const uint32_t abase = (uint32_t)(uintptr_t)(lds_void*)&As[0][0] + 2 * wm * RTM * 32 * RBK;
  const uint32_t wbase = (uint32_t)(uintptr_t)(lds_void*)&Ws[0][0] + 2 * wn * RTN * 32 * RBK;
  constexpr uint32_t A_STAGE = 2 * RBM * RBK, W_STAGE = 2 * RBN * RBK, TILE = 2 * 32 * RBK;

  const int steps = K / RBK;
  bf16x8 fa[2][RTM], fw[2][RTN];
  auto read_operands = [&](int stage, int ks) {
#pragma unroll
    for (int i = 0; i < RTM; ++i) fa[ks][i] = lds_read16(abase + stage * A_STAGE + i * TILE + off[ks]);
#pragma unroll
    for (int j = 0; j < RTN; ++j) fw[ks][j] = lds_read16(wbase + stage * W_STAGE + j * TILE + off[ks]);
  };
  // the MFMAs of MFMA step ks; with MORE, half of the loads of stage s + RING_STAGES - 1 are requested among them,
  // one after a row of MFMAs (requests and arithmetic side by side, not in bursts)
  auto multiply = [&](int ks, auto more, int nstage, int nk0) {
#pragma unroll
    for (int i = 0; i < RTM; ++i) {
#pragma unroll
      for (int j = 0; j < RTN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[ks][i], fw[ks][j], acc[i][j], 0, 0, 0);
      if (decltype(more)::value) {
        constexpr int SLOTS = 2 * RTM;
        const int slot = ks * RTM + i;
#pragma unroll
        for (int t = 0; t < RLA; ++t)
          if ((t * SLOTS) / RLPS == slot) load_a(t, nstage, nk0);
#pragma unroll
        for (int t = 0; t < RLW; ++t)
          if (((RLA + t) * SLOTS) / RLPS == slot) load_w(t, nstage, nk0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // k-step s.  On entry the operands of its first MFMA step are on their way into registers.  The barrier stands
  // between the two MFMA steps: by then this wave has read all it needs of stage s, and once every wave has,
  // stage s + 1 (whose loads were waited for) may be read and the buffer of stage s overwritten (by the loads of
  // k-step s + 1).  So the first operands of k-step s + 1 arrive under the second MFMA step of k-step s.
  static_assert(RING_STAGES == 4 && RLPS % 2 == 0, "the wait counts below are written for four stages and an even number of loads a stage");
  auto step = [&](int s, auto more) {
    const int stage = s % RING_STAGES, nstage = (s + RING_STAGES - 1) % RING_STAGES, nk0 = (s + RING_STAGES - 1) * RBK;
    read_operands(stage, 1);
    lds_wait<RTM + RTN>(fa[0], fw[0]);
    multiply(0, more, nstage, nk0);
    lds_wait<0>(fa[1], fw[1]);
    if (s + 1 < steps) {
      // loads of this wave that may still be on their way: those of stage s + 2, and the half of stage s + 3 just asked for
      if (decltype(more)::value)
        vm_wait<RLPS + RLPS / 2>();
      else if (s + 2 < steps)
        vm_wait<RLPS>();
      else
        vm_wait<0>();
      __builtin_amdgcn_s_barrier();
      read_operands((s + 1) % RING_STAGES, 0);
    }
    multiply(1, more, nstage, nk0);
  };
  using Yes = std::true_type;
  using No = std::false_type;
#pragma unroll
  for (int s = 0; s < RING_STAGES - 1; ++s)
    if (s < steps) {
#pragma unroll
      for (int t = 0; t < RLA; ++t) load_a(t, s, s * RBK);
#pragma unroll
      for (int t = 0; t < RLW; ++t) load_w(t, s, s * RBK);
    }
  if (steps >= 3)
    vm_wait<2 * RLPS>();
  else if (steps == 2)
    vm_wait<RLPS>();
  else
    vm_wait<0>();
  __builtin_amdgcn_s_barrier();
  read_operands(0, 0);
  int s = 0;
  for (; s + RING_STAGES - 1 < steps; ++s) step(s, Yes{});
  for (; s < steps; ++s) step(s, No{});  // the last stages are on their way or have landed: nothing more is requested

  // accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
  if (EPI == EPI_SILU_MUL) {
#pragma unroll
    for (int p = 0; p < RTN / 2; ++p) {
      const int gn = bx * (RBN / 2) + wn * (RTN / 2 * 32) + p * 32 + lane % 32;
      if (gn >= half) continue;
#pragma unroll
      for (int i = 0; i < RTM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int gm = m0 + wm * RTM * 32 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
          const float g = acc[i][2 * p][r], u = acc[i][2 * p + 1][r];
          if (gm < M) c[(size_t)gm * ldc + gn] = (CT)(g / (1.0f + __expf(-g)) * u);
        }
    }
    return;
  }
  if constexpr (EPI == EPI_ACCUMULATE) {
    // as in the tiled kernel: inside C, all old values of a tile are read before any is added to
    if (m0 + (wm + 1) * RTM * 32 <= M && bx * RBN + (wn + 1) * RTN * 32 <= N) {
#pragma unroll
      for (int i = 0; i < RTM; ++i) {
        CT* base = c + (size_t)(m0 + wm * RTM * 32 + i * 32 + 4 * (lane / 32)) * ldc + bx * RBN + wn * RTN * 32 + lane % 32;
        float old[RTN][16];
#pragma unroll
        for (int j = 0; j < RTN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) old[j][r] = (float)base[(size_t)(8 * (r / 4) + r % 4) * ldc + j * 32];
#pragma unroll
        for (int j = 0; j < RTN; ++j)
#pragma unroll
          for (int r = 0; r < 16; ++r) base[(size_t)(8 * (r / 4) + r % 4) * ldc + j * 32] = (CT)(old[j][r] + acc[i][j][r]);
      }
      return;
    }
  }
#pragma unroll
  for (int i = 0; i < RTM; ++i)
#pragma unroll
    for (int j = 0; j < RTN; ++j) {
      const int gn = bx * RBN + wn * RTN * 32 + j * 32 + lane % 32;
      if (gn >= N) continue;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int gm = m0 + wm * RTM * 32 + i * 32 + 8 * (r / 4) + 4 * (lane / 32) + r % 4;
        if (gm < M) store_c<CT>(c + (size_t)gm * ldc + gn, acc[i][j][r], EPI == EPI_ACCUMULATE);
      }
    }
}

// The ring kernel pays where its tiles occupy at least three quarters of the compute units and the loads are whole
// 16-byte pieces.
inline bool ring_takes(const void* a, int lda, const void* w, int ldw, int K) {
  return K % RBK == 0 && K >= RBK * RING_STAGES && lda % 8 == 0 && ldw % 8 == 0 && (uintptr_t)a % 16 == 0 &&
         (uintptr_t)w % 16 == 0;
}
inline bool ring_pays(int epi, const void* a, int lda, const void* w, int ldw, int M, int N, int K) {
  if (!ring_takes(a, lda, w, ldw, K)) return false;
  const int cols = epi == EPI_SILU_MUL ? N / 2 : N, bn = epi == EPI_SILU_MUL ? RBN / 2 : RBN;
  const long long tiles = (long long)((M + RBM - 1) / RBM) * ((cols + bn - 1) / bn);
  return M >= 1024 && tiles >= 192;
}

template <int EPI, typename CT>
int launch_ring(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, hipStream_t stream) {
  const int cols = EPI == EPI_SILU_MUL ? N / 2 : N, bn = EPI == EPI_SILU_MUL ? RBN / 2 : RBN;
  const dim3 grid((cols + bn - 1) / bn, (M + RBM - 1) / RBM), block(RGM * RGN * 64);
  GB_REQUIRE(grid.y <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  hipLaunchKernelGGL((gemm_ring_kernel<EPI, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, 0);
  return launched("gemm_bf16 (ring)");
}

// ----------------------------------------------------------------------- stream
// Products of 17 to a few hundred rows (the mixed steps of serving: a portion of a prompt beside decoded tokens,
// a new turn behind a long history).  They are bound by reading W once, like decoding, but A no longer fits a
// wave's registers; and with the wide tiles above few workgroups exist, each with little on its way from memory
// (a chip-wide 5 TB/s at 2 us of latency wants some 40 KB in flight on every compute unit).
//
// Here a workgroup owns all 128 rows of a row tile and only 32 or 64 rows of W (TN = 1, 2), so that even the QKV
// product of a 2,048-wide model has a workgroup for most compute units without dividing k.  Four waves compute,
// each 32 rows of A by all of the workgroup's columns.  Both operands go from memory straight into LDS
// (global_load_lds, 16 bytes a lane) in k-steps of 64 through two rings: six stages of A (16 KB each; A comes
// from the second-level cache, every workgroup reads the same rows), asked for by the computing waves, and 14 or 7
// stages of W (4 or 8 KB each: some 50 KB on their way from memory per compute unit), asked for by a fifth wave
// that does nothing else.  A wave's loads retire in the order of issue: if one wave asked for both, waiting for
// a stage of A would also wait for every stage of W asked for before it, and W would be three k-steps ahead,
// not thirteen.  A row of a k-step is 128 bytes = 8 pieces; piece p of row r lies at position p ^ (r & 7), which
// spreads the 16-byte operand reads of a wave over all banks.  Waits are written by hand as in the ring kernel.
constexpr int SBK = 64, SBM = 128, SA_STAGES = 6;
// Measured on SmolLM2-1.7B shapes (each product alone, replayed from a graph): up to 64 rows the skinny kernel is as
// fast or faster (it keeps A in registers); from about 200 rows on the wide tiles that divide k are (a workgroup here
// reads two LDS operands for every MFMA); between, this kernel gains 10 to 25 %.
constexpr int STREAM_MAX_ROWS = 128;
// Narrow tiles enough to fill the chip without dividing k.  (128 were taken for enough once: the 4,096 rows of W of a
// Llama-3-8B projection then made 128 workgroups that walk all of k, and its O and down projections of 65 to 128 rows
// took 29 and 81 us where the wide tiles with slices take 14 and 30.)
constexpr int STREAM_FILLS = 192;
// The fewest rows minus one that go to the stream kernel: 48 where it takes the product whole (gate/up of 64 rows:
// SmolLM2-1.7B shapes 23.3 -> 22.0 us, Llama-3-8B shapes 82 -> 73; at 40 rows the wide tiles with slices are as fast or
// faster), 32 where it divides k (the O projection of the 1.7B shapes at 40 to 64 rows 11.4 -> 9.6 us, the down projection
// of the 360M shapes 11.1 -> 9.1).
inline int stream_min_rows(int M, int N, int K, bool silu) {
  const int tiles = ((N + 31) / 32) * ((M + 127) / 128);
  const bool divides = tiles < STREAM_FILLS && K >= 1024 && K < 4096;  // as split_plan decides for the stream kernel's range
  // (other products it would take whole stay with the skinny kernel up to 64 rows, and so does a SiLU-multiply product
  // whose narrow tiles do not fill the chip: SmolLM2-360M's gate/up of 49 to 64 rows 8.7 us there, 10.3 here)
  return divides ? 32 : (silu && tiles >= 2 * STREAM_FILLS) ? 48 : 64;
}
constexpr int SLA = SBM / 8 / 4;  // a computing wave's load instructions per stage of A (an instruction moves 8 rows x 8 pieces)
template <int TN> struct StreamShape {
  static constexpr int BN = 32 * TN, W_STAGES = TN == 1 ? 14 : 7, LW = BN / 8;  // LW: the loading wave's instructions per stage
};

template <int TN, int EPI, typename CT>
__global__ __launch_bounds__(320, 1) void gemm_stream_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w,
                                                             int ldw, CT* __restrict__ c, int ldc, int M, int N, int K,
                                                             int k_slice) {
  using S = StreamShape<TN>;
  constexpr int BN = S::BN, SW = S::W_STAGES, LW = S::LW, DA = SA_STAGES - 1, DW = SW - 1;
  static_assert((DW - 1) * LW < 64 && (DA - 1) * SLA < 64, "a wave counts at most 63 loads on their way");
  if (k_slice > 0) {  // split k: workgroup z of a tile sums its own slice of k into its own copy of C
    const int z = blockIdx.z;
    a += (size_t)z * k_slice;
    w += (size_t)z * k_slice;
    c += (size_t)z * M * ldc;
    K = min(k_slice, K - z * k_slice);
  }
  __shared__ __attribute__((aligned(16))) bf16 As[SA_STAGES][SBM * SBK];
  __shared__ __attribute__((aligned(16))) bf16 Ws[SW][BN * SBK];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int bx = blockIdx.x, m0 = blockIdx.y * SBM;
  const int half = N / 2;  // EPI_SILU_MUL: number of gate rows
  const int steps = K / SBK;
  // Every workgroup of a row tile reads the same rows of A.  If all walked k from 0 they would ask the same few
  // channels of the second-level cache for the same lines at the same time; so each starts somewhere else and
  // walks round (the order of a cell's sum depends on its column tile, never on the rows of the step).
  const int rot = (int)((blockIdx.x * 13u + blockIdx.z * 5u) % (unsigned)steps);
  auto k_of = [&](int step) {
    const int t = step + rot;
    return (t >= steps ? t - steps : t) * SBK;
  };

  if (wave == 4) {
    // ------------------------------------------------------------ the wave that asks for W
    // row of W behind row r of the workgroup's W tile; with EPI_SILU_MUL (TN = 2) the first 32 rows are gate rows
    // and the second 32 the up rows that belong to them; rows beyond N are read from a row that exists
    auto w_row = [&](int r) -> int {
      if (EPI == EPI_SILU_MUL) {
        const int n = bx * 32 + r % 32;
        return n < half ? (r / 32 ? half + n : n) : 0;
      }
      return min(bx * BN + r, N - 1);
    };
    const bf16* wsrc[LW];
#pragma unroll
    for (int t = 0; t < LW; ++t) {
      const int row = t * 8 + lane / 8, piece = (lane % 8) ^ (row & 7);
      wsrc[t] = w + (size_t)w_row(row) * ldw + piece * 8;
    }
    auto load_w = [&](int step) {
#pragma unroll
      for (int t = 0; t < LW; ++t)
        __builtin_amdgcn_global_load_lds((glb_void*)(wsrc[t] + k_of(step)), (lds_void*)&Ws[step % SW][t * 8 * SBK], 16, 0, 2);  // nontemporal: W is read once, in whole 128-byte lines
    };
    for (int t = 0; t < DW && t < steps; ++t) load_w(t);
    // stage 0 has landed once at most the loads asked for after it are on their way
    if (steps >= DW)
      vm_wait<(DW - 1) * LW>();
    else
      vm_wait<0>();
    __builtin_amdgcn_s_barrier();
    for (int s = 0; s < steps; ++s) {
      // everybody has passed the barrier of k-step s - 1: the buffer of stage s - 1 is free
      const bool more = s + DW < steps;
      if (more) load_w(s + DW);
      if (s + 1 < steps) {
        if (more)
          vm_wait<(DW - 1) * LW>();  // stage s + 1 has landed: only what was asked for after it is on its way
        else
          vm_wait<0>();
        __builtin_amdgcn_s_barrier();
      }
    }
    return;
  }

  // ---------------------------------------------------------------- the waves that compute
  // a load instruction moves 8 rows x 8 pieces; rows beyond M are read from a row that exists
  const bf16* asrc[SLA];
#pragma unroll
  for (int t = 0; t < SLA; ++t) {
    const int row = (wave * SLA + t) * 8 + lane / 8, piece = (lane % 8) ^ (row & 7);
    asrc[t] = a + (size_t)min(m0 + row, M - 1) * lda + piece * 8;
  }
  auto load_a = [&](int step) {
#pragma unroll
    for (int t = 0; t < SLA; ++t)
      __builtin_amdgcn_global_load_lds((glb_void*)(asrc[t] + k_of(step)),
                                       (lds_void*)&As[step % SA_STAGES][(wave * SLA + t) * 8 * SBK], 16, 0, 0);
  };
  f32x16 acc[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[j][r] = 0.f;

  // operand of MFMA step kk (0..3): row lane % 32 of a 32-row tile, piece 2 kk + lane / 32
  uint32_t off[4];
#pragma unroll
  for (int kk = 0; kk < 4; ++kk) off[kk] = 2 * ((lane % 32) * SBK + (((2 * kk + lane / 32) ^ (lane & 7)) * 8));
  const uint32_t abase = (uint32_t)(uintptr_t)(lds_void*)&As[0][0] + 2 * wave * 32 * SBK;
  const uint32_t wbase = (uint32_t)(uintptr_t)(lds_void*)&Ws[0][0];
  constexpr uint32_t A_STAGE = 2 * SBM * SBK, W_STAGE = 2 * BN * SBK, TILE = 2 * 32 * SBK;

  bf16x8 fa[2][4], fw[2][4 * TN];  // two sets: the operands of k-step s + 1 arrive under the MFMAs of k-step s
  auto read_operands = [&](int s, int set) {
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      fa[set][kk] = lds_read16(abase + (s % SA_STAGES) * A_STAGE + off[kk]);
#pragma unroll
      for (int j = 0; j < TN; ++j) fw[set][kk * TN + j] = lds_read16(wbase + (s % SW) * W_STAGE + j * TILE + off[kk]);
    }
  };
  using Set0 = std::integral_constant<int, 0>;
  using Set1 = std::integral_constant<int, 1>;

  for (int t = 0; t < DA && t < steps; ++t) load_a(t);
  if (steps >= DA)
    vm_wait<(DA - 1) * SLA>();
  else
    vm_wait<0>();
  __builtin_amdgcn_s_barrier();
  read_operands(0, 0);
  // k-step s, its operands in register set `mine`
  auto step = [&](int s, auto mine) {
    constexpr int set = decltype(mine)::value;
    // everybody has passed the barrier of k-step s - 1: the buffer of stage s - 1 is free
    const bool more = s + DA < steps;
    if (more) load_a(s + DA);
    lds_wait<0>(fa[set], fw[set]);  // all of this wave's reads of stage s have arrived
    if (s + 1 < steps) {
      if (more)
        vm_wait<(DA - 1) * SLA>();  // this wave's part of stage s + 1 has landed
      else
        vm_wait<0>();
      __builtin_amdgcn_s_barrier();
      read_operands(s + 1, set ^ 1);
    }
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int j = 0; j < TN; ++j) acc[j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fa[set][kk], fw[set][kk * TN + j], acc[j], 0, 0, 0);
  };
  for (int s = 0; s < steps; s += 2) {
    step(s, Set0{});
    if (s + 1 < steps) step(s + 1, Set1{});
  }

  // accumulator layout of a 32x32 tile: lane holds column lane%32, rows 8*(r/4) + 4*(lane/32) + r%4
  const int row0 = m0 + wave * 32 + 4 * (lane / 32);
  if (EPI == EPI_SILU_MUL) {
    const int gn = bx * 32 + lane % 32;
    if (gn >= half) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int gm = row0 + 8 * (r / 4) + r % 4;
      const float g = acc[0][r], u = acc[TN - 1][r];
      if (gm < M) c[(size_t)gm * ldc + gn] = (CT)(g / (1.0f + __expf(-g)) * u);
    }
    return;
  }
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int gn = bx * BN + j * 32 + lane % 32;
    if (gn >= N) continue;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int gm = row0 + 8 * (r / 4) + r % 4;
      if (gm < M) store_c<CT>(c + (size_t)gm * ldc + gn, acc[j][r], EPI == EPI_ACCUMULATE);
    }
  }
}

inline bool stream_takes(const void* a, int lda, const void* w, int ldw, int K) {
  return K % SBK == 0 && lda % 8 == 0 && ldw % 8 == 0 && (uintptr_t)a % 16 == 0 && (uintptr_t)w % 16 == 0;
}

template <int EPI, typename CT>
int launch_stream(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, int k_slice, int slices,
                  hipStream_t stream) {
  const int cols = EPI == EPI_SILU_MUL ? N / 2 : N;
  // the SiLU-multiply needs a gate tile and its up tile in one wave; otherwise narrow tiles while they are few
  const int tn = EPI == EPI_SILU_MUL ? 2 : ((cols + 31) / 32) * ((M + SBM - 1) / SBM) * slices > 512 ? 2 : 1;
  const int bn = EPI == EPI_SILU_MUL ? 32 : 32 * tn;
  const dim3 grid((cols + bn - 1) / bn, (M + SBM - 1) / SBM, slices), block(320);
  GB_REQUIRE(grid.y <= 65535 && grid.z <= 65535, "gemm_bf16: M=%d needs more than 65535 row tiles", M);
  if (tn == 2)
    hipLaunchKernelGGL((gemm_stream_kernel<2, EPI, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, k_slice);
  else if constexpr (EPI != EPI_SILU_MUL)
    hipLaunchKernelGGL((gemm_stream_kernel<1, EPI, CT>), grid, block, 0, stream, a, lda, w, ldw, c, ldc, M, N, K, k_slice);
  return launched("gemm_bf16 (stream)");
}

// ------------------------------------------------------------------------ split k
// A product with few tiles (17 to a few hundred rows, or few rows of W) leaves most compute units idle
// and, as a skinny product, makes every workgroup read all of A.  Here the tiled kernel's workgroups
// also divide k: workgroup (tile, z) sums slice z of k into copy z of a float32 C in a workspace, and a
// second kernel adds the copies in the order of z and applies the epilogue.  Tiles of 64 or 128 rows; with
// a thousand rows and more and a long k, the ring kernel's tiles of 256.
struct SplitPlan {
  int bm, slices, k_slice;
  size_t floats;  // of workspace
  bool ring;      // the ring kernel's 256 x 256 tiles, if the operands allow (else the tiled kernel's, same slices)
  bool stream;    // the stream kernel's 128 x 32 tiles, if the operands allow (else the tiled kernel's, same slices)
};

inline SplitPlan split_plan(int M, int N, int K, bool silu = false) {
  SplitPlan p{M <= 64 ? 64 : 128, 1, 0, 0, false, false};
  // many rows, a long k and few 256 x 256 tiles (the down projection of a prompt portion): slices of k fill the
  // chip with the ring kernel's tiles once; a slice keeps 1,024 of k or more
  if (M >= 1024 && K >= 4096 && K % TBK == 0 && N % 8 == 0) {
    const int tiles = ((M + RBM - 1) / RBM) * ((N + RBN - 1) / RBN);
    int want = tiles < 192 ? 256 / tiles : 1;
    if (want > K / 1024) want = K / 1024;
    if (want >= 2) {
      p.k_slice = ((K + want - 1) / want + TBK - 1) / TBK * TBK;
      p.slices = (K + p.k_slice - 1) / p.k_slice;
      if (p.slices >= 2 && K - (p.slices - 1) * p.k_slice >= RBK * RING_STAGES) {
        p.floats = (size_t)p.slices * M * N;
        p.ring = true;
        return p;
      }
      p.slices = 1, p.k_slice = 0;
    }
  }
  if (M > stream_min_rows(M, N, K, silu) && M <= STREAM_MAX_ROWS && K % SBK == 0 && N % 8 == 0) {
    // the stream kernel's range: its tiles are narrow, so only products with few rows of W divide k at all
    // (the O and down projections); a slice keeps 512 of k or more
    const int tiles = ((N + 31) / 32) * ((M + SBM - 1) / SBM);
    if (tiles >= STREAM_FILLS) return p;  // enough narrow tiles: no slices at all
    if (K < 4096) {              // a long k (the down projection) is left to the wide tiles' slices below: measured faster
      int want = (256 + tiles - 1) / tiles;
      if (want > K / 512) want = K / 512;
      if (want < 2) return p;
      p.k_slice = ((K + want - 1) / want + SBK - 1) / SBK * SBK;
      p.slices = (K + p.k_slice - 1) / p.k_slice;
      if (p.slices < 2) return SplitPlan{p.bm, 1, 0, 0, false, false};
      p.floats = (size_t)p.slices * M * N;
      p.stream = true;
      return p;
    }
  }
  const int tiles = ((N + 127) / 128) * ((M + p.bm - 1) / p.bm);
  if (tiles >= 192 || N % 8 != 0) return p;
  // measured on SmolLM2-1.7B shapes: a long k (the down projection) always gains; a short one where the
  // skinny kernel is at its weakest (33 to 64 rows: every workgroup reads all of A) and where the tiles are
  // very few (the O projection of a portion of some hundred rows: 16 to 64 tiles)
  if (K < 4096 && !(M > 32 && M <= 64) && !(M > 64 && K >= 2048 && tiles <= 128)) return p;
  // a slice keeps at least 8 k-steps (shorter ones cost more in partial sums than they gain), and of a long k, beyond
  // 64 rows, 16 k-steps: a workgroup of 128 rows has more to do in a k-step, and the pass that adds the slices reads
  // half as much (same box: the down projection of 256 rows on SmolLM2-1.7B shapes 26.7 -> 24.2 us, of 384 rows
  // 36.0 -> 30.6; Llama-3-8B's QKV of 192 to 256 rows 36-38 -> 31, its O projection 25-26 -> 23-24)
  int want = (512 + tiles - 1) / tiles;
  want = want > 16 ? 16 : want;
  if (M > 64 && K >= 4096 && want > K / (16 * TBK)) want = K / (16 * TBK);
  if (want > K / (8 * TBK)) want = K / (8 * TBK);
  if (want < 2) return p;
  p.k_slice = ((K + want - 1) / want + TBK - 1) / TBK * TBK;
  p.slices = (K + p.k_slice - 1) / p.k_slice;
  if (p.slices < 2) return SplitPlan{p.bm, 1, 0, 0, false, false};
  p.floats = (size_t)p.slices * M * N;
  // tiles of 64 rows where even with the slices a third of the compute units would have no workgroup
  if (tiles * p.slices < 168) p.bm = 64;
  return p;
}

// ws: [slices][M][N] float32.  Four columns a thread; EPI_SILU_MUL pairs column j with column N/2 + j.
template <int EPI, typename CT>
__global__ void splitk_reduce_kernel(const float* __restrict__ ws, int slices, CT* __restrict__ c, int ldc, int M, int N) {
  const int cols = EPI == EPI_SILU_MUL ? N / 2 : N, groups = cols / 4;
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)M * groups) return;
  const int m = (int)(idx / groups), j = (int)(idx % groups) * 4;
  f32x4 sum = {0.f, 0.f, 0.f, 0.f}, up = {0.f, 0.f, 0.f, 0.f};
  const size_t copy = (size_t)M * N;  // floats between one slice's copy of C and the next
  const float* row = ws + (size_t)m * N;
  int z = 0;
  for (; z + 4 <= slices; z += 4) {  // four slices' loads are on their way together; the sums keep the order of z
    f32x4 v[4], u[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      v[t] = *reinterpret_cast<const f32x4*>(row + (z + t) * copy + j);
      if (EPI == EPI_SILU_MUL) u[t] = *reinterpret_cast<const f32x4*>(row + (z + t) * copy + N / 2 + j);
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
      sum += v[t];
      if (EPI == EPI_SILU_MUL) up += u[t];
    }
  }
  for (; z < slices; ++z) {
    sum += *reinterpret_cast<const f32x4*>(row + z * copy + j);
    if (EPI == EPI_SILU_MUL) up += *reinterpret_cast<const f32x4*>(row + z * copy + N / 2 + j);
  }
  CT* out = c + (size_t)m * ldc + j;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    float v = sum[e];
    if (EPI == EPI_SILU_MUL) v = v / (1.0f + __expf(-v)) * up[e];
    store_c<CT>(out + e, v, EPI == EPI_ACCUMULATE);
  }
}

// The same pass for a product that accumulates into the float32 residual, one workgroup a row; with the new row
// in hand it also does the RMS norm that reads the residual next: h[m, n] = gamma[n] * (r[m, n] * s),
// s = 1 / sqrt(mean(r[m]^2) + eps), the formula of the norm's own kernel.  Rows of up to SPLIT_NORM_MAX columns.
constexpr int SPLIT_NORM_MAX = 256 * 4 * 8;
template <typename G>
__global__ __launch_bounds__(256) void splitk_reduce_norm_kernel(const float* __restrict__ ws, int slices, float* __restrict__ c,
                                                                 int ldc, int M, int N, const G* __restrict__ gamma, float eps,
                                                                 bf16* __restrict__ h, int ldh) {
  __shared__ float partial[4];
  const int m = blockIdx.x, tid = threadIdx.x;
  f32x4 r[8];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = (tid + 256 * i) * 4;
    if (j >= N) break;
    f32x4 sum = {0.f, 0.f, 0.f, 0.f};  // the slices in their order, then the residual: as the plain second pass does
    const size_t copy = (size_t)M * N;
    const float* row = ws + (size_t)m * N + j;
    const f32x4 old = *reinterpret_cast<const f32x4*>(c + (size_t)m * ldc + j);
    int z = 0;
    for (; z + 4 <= slices; z += 4) {  // four slices' loads on their way together
      f32x4 v[4];
#pragma unroll
      for (int t = 0; t < 4; ++t) v[t] = *reinterpret_cast<const f32x4*>(row + (z + t) * copy);
#pragma unroll
      for (int t = 0; t < 4; ++t) sum += v[t];
    }
    for (; z < slices; ++z) sum += *reinterpret_cast<const f32x4*>(row + z * copy);
    sum = old + sum;
    *reinterpret_cast<f32x4*>(c + (size_t)m * ldc + j) = sum;
    r[i] = sum;
    ss += sum[0] * sum[0] + sum[1] * sum[1] + sum[2] * sum[2] + sum[3] * sum[3];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off, 64);
  if (tid % 64 == 0) partial[tid / 64] = ss;
  __syncthreads();
  const float total = partial[0] + partial[1] + partial[2] + partial[3];
  const float scale = 1.0f / sqrtf(total / (float)N + eps);
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int j = (tid + 256 * i) * 4;
    if (j >= N) break;
    bf16x4 o;
#pragma unroll
    for (int e = 0; e < 4; ++e) o[e] = (bf16)((float)gamma[j + e] * (r[i][e] * scale));
    *reinterpret_cast<bf16x4*>(h + (size_t)m * ldh + j) = o;
  }
}

// Folded tiles pay when the product has at most 8 rows and whole tiles of 16 rows of W would leave
// compute units without a workgroup (measured: with 384 such tiles they no longer do).
inline bool fold_pays(int M, int N) { return M <= 8 && (N + 15) / 16 < 256; }

// What an accumulating product of these sizes can do for the RMS norm that reads the residual after it:
// 0 nothing; 1 (the folded kernel for at most 8 rows, the skinny kernel up to 64) the operand bf16(gamma * r) and
// partial sums, see NormExtras;
// 2 (a product that divides k, given its workspace) the whole norm, in the pass that adds the slices.
inline int emit_mode(int M, int N, int K) {
  if (fold_pays(M, N)) return 1;
  if (M > 16 && N % 4 == 0 && N <= SPLIT_NORM_MAX && split_plan(M, N, K).slices > 1) return 2;
  if (M <= 64 && !(M > 16 && N >= 32768)) return 1;  // the skinny kernel
  return 0;
}
// Tiles of columns for which an emitting product of these sizes writes partial sums.
inline int emit_parts(int M, int N) {
  if (fold_pays(M, N)) return (N + 7) / 8;
  if (M > 64) return 0;
  return (N + 15) / 16 < 256 ? (N + 7) / 8 : (N + 15) / 16;  // the skinny kernel: half tiles while the tiles are few
}

template <int EPI, typename CT>
int launch_split(const bf16* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, float* ws,
                 const SplitPlan& plan, hipStream_t stream, const NormExtras* norm = nullptr, float eps = 0.f) {
  const dim3 grid((N + 127) / 128, (M + plan.bm - 1) / plan.bm, plan.slices), block(256);
  const bool kfull = K % TBK == 0;
  const bool ring = plan.ring && ring_takes(a, lda, w, ldw, K);
  const bool streams = plan.stream && stream_takes(a, lda, w, ldw, K);
  if (streams) {
    if (int rc = launch_stream<EPI_STORE, float>(a, lda, w, ldw, ws, N, M, N, K, plan.k_slice, plan.slices, stream)) return rc;
  }
  if (ring)
    hipLaunchKernelGGL((gemm_ring_kernel<EPI_STORE, float>), dim3((N + RBN - 1) / RBN, (M + RBM - 1) / RBM, plan.slices), dim3(RGM * RGN * 64),
                       0, stream, a, lda, w, ldw, ws, N, M, N, K, plan.k_slice);
#define GB_S(WM, FULL)                                                                                                   \
  if (!ring && !streams && (plan.bm == 64 * WM) && kfull == FULL)                                                                   \
    hipLaunchKernelGGL((gemm_tiled_kernel<WM, 2, 1, EPI_STORE, FULL, float>), grid, block, 0, stream, a, lda, w, ldw, ws, \
                       N, M, N, K, plan.k_slice);
  GB_S(1, true) GB_S(1, false) GB_S(2, true) GB_S(2, false)
#undef GB_S
  if (int rc = launched("gemm_bf16 (split k)")) return rc;
  if constexpr (EPI == EPI_ACCUMULATE && std::is_same<CT, float>::value) {
    if (norm && norm->emit_h) {
      if (norm->emit_gamma_f32)
        hipLaunchKernelGGL((splitk_reduce_norm_kernel<float>), dim3(M), dim3(256), 0, stream, ws, plan.slices, c, ldc, M, N,
                           (const float*)norm->emit_gamma, eps, norm->emit_h, norm->emit_ldh);
      else
        hipLaunchKernelGGL((splitk_reduce_norm_kernel<bf16>), dim3(M), dim3(256), 0, stream, ws, plan.slices, c, ldc, M, N,
                           (const bf16*)norm->emit_gamma, eps, norm->emit_h, norm->emit_ldh);
      return launched("gemm_bf16 (split k, second pass with the norm)");
    }
  }
  const int cols = EPI == EPI_SILU_MUL ? N / 2 : N;
  const size_t threads = (size_t)M * (cols / 4);
  hipLaunchKernelGGL((splitk_reduce_kernel<EPI, CT>), dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, stream, ws,
                     plan.slices, c, ldc, M, N);
  return launched("gemm_bf16 (split k, second pass)");
}

// ------------------------------------------------------------------------ skinny
// grid (row tiles of W).  A workgroup of WAVES waves owns 16 rows of W and walks all of k in slices
// of ITERS*WAVES*64: wave w takes the 64-wide k blocks w, w+WAVES, ... of a slice; inside a block
// lane group q holds k = 8q..8q+7 of each half of 32 (the same split for W and for A, so the
// products pair up).  All loads of a slice are issued before its first MFMA.  The waves combine
// through LDS in wave order.  Few rows of W (a small N) are given many waves each, so that the
// launch still keeps enough loads in flight to use the memory system; no partial result ever
// leaves the workgroup, so no pass over memory is needed to combine them.
//
// EPI_STORE / EPI_ACCUMULATE: C[m, n] = or += the product.  EPI_SILU_MUL: W holds gate rows
// [0, N/2) and up rows [N/2, N); a tile takes 8 gate rows and the 8 up rows that belong to them
// and writes act[m, j] = gate / (1 + exp(-gate)) * up (crates/glassbox-core/src/model.rs:336-340)
// to C[M, N/2].

// The A operand of one lane: 8 consecutive k of row m.  Plain: bfloat16 rows as they are.  RMS: the
// rows are the float32 residual; the operand is bf16(gamma[k] * x[k]) and sum(x^2) is gathered on
// the way, so that the caller can scale the finished product by 1/sqrt(mean(x^2) + eps): the RMS
// norm (crates/glassbox-core/src/model.rs:94-100) without a pass of its own.
// The 16 bytes that lane `lane` of the wave holds in v.
__device__ __forceinline__ bf16x8 from_lane(bf16x8 v, int lane) {
  typedef int i32x4 __attribute__((ext_vector_type(4)));
  i32x4 w = __builtin_bit_cast(i32x4, v);
#pragma unroll
  for (int i = 0; i < 4; ++i) w[i] = __builtin_amdgcn_ds_bpermute(lane * 4, w[i]);
  return __builtin_bit_cast(bf16x8, w);
}

template <bool RMS>
__device__ __forceinline__ bf16x8 load_a(const void* a, int lda, int m, int k, bool ok, const void* gamma, int gamma_f32,
                                         float& ss) {
  if (!ok) return zero8();
  if (!RMS) return load8((const bf16*)a + (size_t)m * lda + k);
  const float* x = (const float*)a + (size_t)m * lda + k;
  const f32x4 x0 = *reinterpret_cast<const f32x4*>(x), x1 = *reinterpret_cast<const f32x4*>(x + 4);
  float g[8];
  if (gamma_f32) {
    const f32x4 g0 = *reinterpret_cast<const f32x4*>((const float*)gamma + k);
    const f32x4 g1 = *reinterpret_cast<const f32x4*>((const float*)gamma + k + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      g[e] = g0[e];
      g[4 + e] = g1[e];
    }
  } else {
    const bf16x8 gb = load8((const bf16*)gamma + k);
#pragma unroll
    for (int e = 0; e < 8; ++e) g[e] = (float)gb[e];
  }
  bf16x8 out;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float xe = e < 4 ? x0[e] : x1[e - 4];
    ss += xe * xe;
    out[e] = (bf16)(g[e] * xe);
  }
  return out;
}

// (Up to 16 rows, sixteen waves, two row tiles and two loads in flight: the kernel needs exactly 64 registers a lane,
// with which two workgroups share a compute unit, one's loads on their way while the other adds up and stores.  One
// register more and only one fits: decode steps of one to eight requests were 4 % slower.)
template <int MT, int WAVES, int ITERS, int RT, int EPI, bool RMS, typename CT, bool HALF = false>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const void* __restrict__ a, int lda,
                                                                 const bf16* __restrict__ w, int ldw, CT* __restrict__ c,
                                                                 int ldc, int M, int N, int K, const void* __restrict__ gamma,
                                                                 int gamma_f32, float eps, NormExtras extra, RopeExtras rope) {
  __shared__ float part[WAVES][RT][MT][64][4];
  __shared__ float sspart[RMS ? WAVES : 1][MT][64];
  constexpr int PJ = WAVES * 64 / (MT * 16) < 64 ? WAVES * 64 / (MT * 16) : 64;  // threads that share a row's partial sums
  __shared__ float red[RMS ? 1 : PJ][MT * 16];  // (with RMS the rows bring no partial sums)
  __shared__ float emit_sq[4][RT][MT][16];
  const float* __restrict__ parts = extra.parts;
  const int n_parts = extra.n_parts;
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  // Partial sums of squares of the rows, one per tile of the product that made them: some threads a row add up
  // every so-manieth, the epilogue adds up theirs, both in a fixed order.  Up to 8 rows (8 floats a tile): J8 threads a
  // row, few terms each.  Beyond (64 floats a tile): PJ threads a row, and where a thread has many terms, four loads
  // at a time are asked for before any is added (one after the other they would each wait).  The first form is kept
  // as it is on purpose: with it the sixteen-wave kernel needs 64 registers and fits twice on a compute unit, with
  // the general form alone the compiler keeps one or two more through the main loop.
  constexpr int J8 = WAVES * 8 < 64 ? WAVES * 8 : 64;
  float* red8 = &red[0][0];  // [J8][8]
  if (!RMS && parts != nullptr) {
    if (M <= 8) {
      for (int t = tid; t < 8 * J8; t += WAVES * 64) {
        const int m = t & 7, j = t >> 3;
        float sum = 0.f;
        for (int p = j; p < n_parts; p += J8) sum += parts[p * 8 + m];
        red8[j * 8 + m] = sum;
      }
    } else {
      const int m = tid % (MT * 16), j = tid / (MT * 16);
      float sum = 0.f;
      if (m < M && j < PJ)
        for (int p = j; p < n_parts; p += 4 * PJ) {
          float got[4];
#pragma unroll
          for (int u = 0; u < 4; ++u) got[u] = p + u * PJ < n_parts ? parts[(p + u * PJ) * 64 + m] : 0.f;
#pragma unroll
          for (int u = 0; u < 4; ++u) sum += got[u];
        }
      if (j < PJ) red[j][m] = sum;
    }
  }
  const bf16* wrow[RT];
  bool row_ok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    int tile = blockIdx.x * RT + rt, pair_lo = 0, pair_hi = 8;
    if (EPI == EPI_ROPE && RT == 2 && rope.three_halves) tile = three_halves_tile(blockIdx.x, rt, &pair_lo, &pair_hi);
    int row;
    if (EPI == EPI_SILU_MUL) {
      row = r < 8 ? tile * 8 + r : N / 2 + tile * 8 + (r - 8);
    } else if (EPI == EPI_ROPE) {
      // a tile is 8 pairs of one head: its dims d0..d0+7 and those hd/2 further on
      const int per_head = rope.hd / 16, head = tile / per_head, d0 = (tile % per_head) * 8;
      row = head * rope.hd + (r < 8 ? d0 + r : rope.hd / 2 + d0 + (r - 8));
    } else if (HALF) {
      row = tile * 8 + (r & 7);  // a workgroup owns 8 rows of W: the tile's lower half stays empty
    } else {
      row = tile * 16 + r;
    }
    row_ok[rt] = EPI == EPI_SILU_MUL ? (tile * 8 + (r & 7) < N / 2) : HALF ? (r < 8 && row < N) : row < N;
    if (EPI == EPI_ROPE) row_ok[rt] = row_ok[rt] && (r & 7) >= pair_lo && (r & 7) < pair_hi;
    wrow[rt] = w + (size_t)(row_ok[rt] ? row : 0) * ldw;
  }

  f32x4 acc[RT][MT];
  float ss[MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    ss[t] = 0.f;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int e = 0; e < 4; ++e) acc[rt][t][e] = 0.f;
  }

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
      bf16x8 xf[ITERS][2];
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int k = kbeg + (wave + WAVES * it) * 64 + q * 8;
        xf[it][0] = load_a<RMS>(a, lda, r, k, r < M && k < K, gamma, gamma_f32, ss[0]);
        xf[it][1] = load_a<RMS>(a, lda, r, k + 32, r < M && k + 32 < K, gamma, gamma_f32, ss[0]);
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
          bf16x8 x0, x1;
          if (RMS) {
            const int m = t * 16 + r;
            x0 = load_a<RMS>(a, lda, m, k, m < M && k < K, gamma, gamma_f32, ss[t]);
            x1 = load_a<RMS>(a, lda, m, k + 32, m < M && k + 32 < K, gamma, gamma_f32, ss[t]);
          } else {
            // With several column blocks the rows of A are as much traffic from the cache as W is from memory, and the
            // cache serves a wave's load faster when neighbouring lanes share a piece of 64 bytes than when each asks
            // for 16 bytes of another row: lane 4R + Q loads piece Q of row R, and the operand's lane (row lane%16,
            // piece lane/16) takes it from there through the LDS crossbar.
            const int m = t * 16 + (lane >> 2), ka = k - q * 8 + (lane & 3) * 8;
            const bf16x8 y0 = load_a<false>(a, lda, m, ka, m < M && ka < K, gamma, gamma_f32, ss[t]);
            const bf16x8 y1 = load_a<false>(a, lda, m, ka + 32, m < M && ka + 32 < K, gamma, gamma_f32, ss[t]);
            x0 = from_lane(y0, 4 * r + q);
            x1 = from_lane(y1, 4 * r + q);
          }
#pragma unroll
          for (int rt = 0; rt < RT; ++rt) {
            acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][0], x0, acc[rt][t], 0, 0, 0);
            acc[rt][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][1], x1, acc[rt][t], 0, 0, 0);
          }
        }
      }
    }
  }
  // D[n, m]: lane l holds column m = l%16 and rows n = 4*(l/16) + e.  The first 256 threads own the
  // cells of the tiles: thread tid owns cell (l = tid/4, e = tid%4) of every row tile and column block.
  const int l = (tid % 256) / 4, e = tid % 4;
  const int nrow = 4 * (l / 16) + e;  // row of the tile, 0..15
  // What the owners will need from memory at the end (a cell's old value and the gamma of a norm to prepare; a
  // row's cosine, sine and cache slot) is asked for here, before the waves meet, so that it arrives while they do.
  constexpr int ROWS = HALF ? 8 : 16;  // rows of W a tile owns
  const bool emits = EPI == EPI_ACCUMULATE && extra.emit_h != nullptr;
  const bool empty = HALF && nrow >= 8;  // the lower half of a half tile
  float old[RT][MT], emit_g[RT], cs[RT][MT], sn[RT][MT];
  int slot[MT];
  if (EPI == EPI_ACCUMULATE && tid < 256) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n = (blockIdx.x * RT + rt) * ROWS + nrow;
      emit_g[rt] = 0.f;
      if (emits && !empty && n < N)
        emit_g[rt] = extra.emit_gamma_f32 ? ((const float*)extra.emit_gamma)[n] : (float)((const bf16*)extra.emit_gamma)[n];
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + l % 16;
        old[rt][t] = (!empty && m < M && n < N) ? (float)c[(size_t)m * ldc + n] : 0.f;
      }
    }
  }
  constexpr bool ROPE_EARLY = MT * RT <= 4;  // beyond that the registers would not hold what is asked for early
  if (EPI == EPI_ROPE && ROPE_EARLY && tid < 256) {
#pragma unroll
    for (int t = 0; t < MT; ++t) {
      const int m = t * 16 + l % 16;
      slot[t] = (rope.slots != nullptr && m < M) ? rope.slots[m] : 0;
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        int tile = blockIdx.x * RT + rt, pair_lo = 0, pair_hi = 8;
        if (RT == 2 && rope.three_halves) tile = three_halves_tile(blockIdx.x, rt, &pair_lo, &pair_hi);
        const int pair = (tile % (rope.hd / 16)) * 8 + (nrow & 7);
        const bool rotated = rope.cosv != nullptr && m < M && tile / (rope.hd / 16) < rope.nh + rope.nkv;
        cs[rt][t] = rotated ? rope.cosv[(size_t)m * (rope.hd / 2) + pair] : 1.f;
        sn[rt][t] = rotated ? rope.sinv[(size_t)m * (rope.hd / 2) + pair] : 0.f;
      }
    }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int t = 0; t < MT; ++t)
#pragma unroll
      for (int e = 0; e < 4; ++e) part[wave][rt][t][lane][e] = acc[rt][t][e];
  if (RMS) {
#pragma unroll
    for (int t = 0; t < MT; ++t) sspart[wave][t][lane] = ss[t];
  }
  __syncthreads();
  if (tid >= 256) return;

  float v[RT][MT];
#pragma unroll
  for (int t = 0; t < MT; ++t) {
    float scale = 1.f;
    if (RMS) {
      // sum(x^2) of row m = t*16 + l%16: its k were spread over the waves and over the four lane groups
      float tot = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
        for (int qq = 0; qq < 4; ++qq) tot += sspart[wv][t][l % 16 + 16 * qq];
      scale = 1.0f / sqrtf(tot / (float)K + eps);
    } else if (parts != nullptr) {
      float tot = 0.f;
      if (M <= 8) {
        if (l % 16 < 8) {
#pragma unroll 8
          for (int j = 0; j < J8; ++j) tot += red8[j * 8 + l % 16];
        }
      } else {
#pragma unroll 8
        for (int j = 0; j < PJ; ++j) tot += red[j][t * 16 + l % 16];
      }
      scale = 1.0f / sqrtf(tot / (float)K + eps);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float s = part[0][rt][t][l][e];
#pragma unroll
      for (int wv = 1; wv < WAVES; ++wv) s += part[wv][rt][t][l][e];
      v[rt][t] = s * scale;
    }
  }
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
  } else if (EPI == EPI_ROPE) {
    // rows 0..7 and 8..15 of a tile are each other's partners: they meet through LDS as gate and up do
    float* other = &part[WAVES - 1][0][0][0][0];
    __syncthreads();
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int t = 0; t < MT; ++t) other[(rt * MT + t) * 256 + tid] = v[rt][t];
    __syncthreads();
    const int half = rope.hd / 2, per_head = rope.hd / 16;
    const bool upper = nrow >= 8;
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      int tile = blockIdx.x * RT + rt, pair_lo = 0, pair_hi = 8;
      if (RT == 2 && rope.three_halves) tile = three_halves_tile(blockIdx.x, rt, &pair_lo, &pair_hi);
      if ((nrow & 7) < pair_lo || (nrow & 7) >= pair_hi) continue;
      const int head = tile / per_head, pair = (tile % per_head) * 8 + (nrow & 7);
      const int dim = upper ? half + pair : pair;
      if (head * rope.hd + dim >= N) continue;
      const bool is_value = head >= rope.nh + rope.nkv, is_key = head >= rope.nh && !is_value;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + l % 16;
        if (m >= M) continue;
        float y = v[rt][t];
        if (!is_value && rope.cosv != nullptr) {
          const float p = other[(rt * MT + t) * 256 + (tid ^ 128)];
          const float co = ROPE_EARLY ? cs[rt][t] : rope.cosv[(size_t)m * half + pair];
          const float si = ROPE_EARLY ? sn[rt][t] : rope.sinv[(size_t)m * half + pair];
          y = upper ? y * co + p * si : y * co - p * si;
        }
        const bf16 yb = (bf16)y;
        c[(size_t)m * ldc + head * rope.hd + dim] = (CT)yb;
        if (rope.slots != nullptr && head >= rope.nh) {
          const int sl = ROPE_EARLY ? slot[t] : rope.slots[m], page = sl / rope.page_size, off = sl % rope.page_size;
          if (is_key)
            rope.k_pages[((size_t)page * rope.nkv + (head - rope.nh)) * rope.page_size * rope.hd +
                         key_offset(off, dim, rope.page_size, 8)] = yb;  // hd is a multiple of 16: pieces of 8
          else
            rope.v_pages[(((size_t)page * rope.nkv + (head - rope.nh - rope.nkv)) * rope.hd + dim) * rope.page_size + off] = yb;
        }
      }
    }
  } else {
    // accumulating onto the old values asked for above
    if (empty && !emits) return;
    float sq[RT][MT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const int n = (blockIdx.x * RT + rt) * ROWS + nrow;
#pragma unroll
      for (int t = 0; t < MT; ++t) {
        const int m = t * 16 + l % 16;
        sq[rt][t] = 0.f;
        if (!empty && m < M && n < N) {
          const float now = EPI == EPI_ACCUMULATE ? old[rt][t] + v[rt][t] : v[rt][t];
          c[(size_t)m * ldc + n] = (CT)now;
          if (emits) {
            extra.emit_h[(size_t)m * extra.emit_ldh + n] = (bf16)(emit_g[rt] * now);
            sq[rt][t] = now * now;
          }
        }
      }
    }
    if (emits) {
      // sum of squares over a tile's columns, per row: a row's 16 cells lie in four neighbouring lanes of each of
      // the four waves that are still here; added in a fixed order
#pragma unroll
      for (int rt = 0; rt < RT; ++rt)
#pragma unroll
        for (int t = 0; t < MT; ++t) {
          float x = sq[rt][t];
          x += __shfl_xor(x, 1, kWave);
          x += __shfl_xor(x, 2, kWave);
          if (e == 0) emit_sq[wave][rt][t][l % 16] = x;
        }
      __syncthreads();  // the four waves that are still here
      const int stride = parts_stride(M);
      for (int i = tid; i < RT * MT * 16; i += 256) {
        const int rt = i / (MT * 16), t = i / 16 % MT, mm = i % 16, m = t * 16 + mm;
        const float tot = emit_sq[0][rt][t][mm] + emit_sq[1][rt][t][mm] + emit_sq[2][rt][t][mm] + emit_sq[3][rt][t][mm];
        if (m < M) extra.emit_ss[(size_t)(blockIdx.x * RT + rt) * stride + m] = tot;
      }
    }
  }
}

// ------------------------------------------------------------------------ folded (M <= 8)
// With at most 8 rows of A, a 16 x 16 tile has room for two k ranges side by side.  Rows 0..7 of the
// tile are 8 rows of W over one part of a 128-wide k block (k 0..31 and 64..95 of it) and rows 8..15 the same
// 8 rows of W over the other (k 32..63 and 96..127); columns 0..7 are the rows of A over the first part,
// columns 8..15 over the second.  Cells (n, m) and (n + 8, m + 8) then hold the two halves of one sum; the other two
// quarters of the tile pair the wrong halves and are dropped.  A workgroup so owns 8 rows of W, not
// 16, and a product with few rows of W (decoding: the O and down projections) has a workgroup for
// every compute unit: one compute unit draws only a fraction of the memory bandwidth.  The halves of a lane's two
// loads are chosen so that one load instruction of the wave reads whole 128-byte lines of its 8 rows (k 0..63 of
// the block, then 64..127), and the loads are nontemporal: W is read once (the down projection of the
// SmolLM2-1.7B shapes at 8 rows 11.0 -> 10.3 us, the O projection 5.1 -> 4.7; with half lines an instruction,
// nontemporal loads were slower than plain ones).
template <int WAVES, int ITERS, int RT, int EPI, bool RMS, typename CT>
__global__ __launch_bounds__(WAVES * 64) void gemm_fold_kernel(const void* __restrict__ a, int lda,
                                                               const bf16* __restrict__ w, int ldw, CT* __restrict__ c,
                                                               int ldc, int M, int N, int K, const void* __restrict__ gamma,
                                                               int gamma_f32, float eps, NormExtras extra) {
  static_assert(EPI != EPI_SILU_MUL && WAVES >= 4, "folded tiles store or accumulate; the first four waves finish");
  __shared__ float part[WAVES][RT][64][4];
  __shared__ float sspart[RMS ? WAVES : 1][64];
  __shared__ float squares[RT][8][8];
  const int tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int r = lane % 16, q = lane / 16;
  const int r8 = r & 7, khalf = (r >> 3) * 32;  // row of W and of A; which quarter of a k block: a load of the wave reads whole 128-byte lines
  const bf16* wrow[RT];
  bool row_ok[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int row = (blockIdx.x * RT + rt) * 8 + r8;
    row_ok[rt] = row < N;
    wrow[rt] = w + (size_t)(row_ok[rt] ? row : 0) * ldw;
  }
  f32x4 acc[RT];
  float ss = 0.f;
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int e = 0; e < 4; ++e) acc[rt][e] = 0.f;

  // D[n, m]: lane l holds column m = l%16 and rows n = 4*(l/16) + e; thread tid of the first four waves owns cell
  // (l = tid/4, e = tid%4) at the end.  What it will need from memory then (the cell's old value, the gamma of a norm
  // to prepare) is asked for now, so that it arrives under the stream of W and not after it.
  const int l = (tid % 256) / 4, e = tid % 4;
  const int nrow = 4 * (l / 16) + e, m = l % 16;
  const bool emits = EPI == EPI_ACCUMULATE && extra.emit_h != nullptr;
  const bool mine = tid < 256 && nrow < 8 && m < 8;
  float old[RT], emit_g[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int n = (blockIdx.x * RT + rt) * 8 + nrow;
    old[rt] = emit_g[rt] = 0.f;
    if (mine && m < M && n < N) {
      if (EPI == EPI_ACCUMULATE) old[rt] = (float)c[(size_t)m * ldc + n];
      if (emits) emit_g[rt] = extra.emit_gamma_f32 ? ((const float*)extra.emit_gamma)[n] : (float)((const bf16*)extra.emit_gamma)[n];
    }
  }

  for (int kbeg = 0; kbeg < K; kbeg += ITERS * WAVES * 128) {
    bf16x8 wf[RT][ITERS][2], xf[ITERS][2];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int it = 0; it < ITERS; ++it) {
        const int k = kbeg + (wave + WAVES * it) * 128 + khalf + q * 8;
        wf[rt][it][0] = (row_ok[rt] && k < K) ? load8_once(wrow[rt] + k) : zero8();
        wf[rt][it][1] = (row_ok[rt] && k + 64 < K) ? load8_once(wrow[rt] + k + 64) : zero8();
      }
#pragma unroll
    for (int it = 0; it < ITERS; ++it) {
      const int k = kbeg + (wave + WAVES * it) * 128 + khalf + q * 8;
      xf[it][0] = load_a<RMS>(a, lda, r8, k, r8 < M && k < K, gamma, gamma_f32, ss);
      xf[it][1] = load_a<RMS>(a, lda, r8, k + 64, r8 < M && k + 64 < K, gamma, gamma_f32, ss);
    }
#pragma unroll
    for (int it = 0; it < ITERS; ++it)
#pragma unroll
      for (int rt = 0; rt < RT; ++rt) {
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][0], xf[it][0], acc[rt], 0, 0, 0);
        acc[rt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[rt][it][1], xf[it][1], acc[rt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int e = 0; e < 4; ++e) part[wave][rt][lane][e] = acc[rt][e];
  if (RMS) sspart[wave][lane] = ss;
  __syncthreads();
  if (tid >= 256) return;
  if (!mine && !emits) return;
  float scale = 1.f;
  if (RMS && mine) {
    // sum(x^2) of row m: its k were spread over the waves, the four lane groups and the two halves
    float tot = 0.f;
#pragma unroll
    for (int wv = 0; wv < WAVES; ++wv)
#pragma unroll
      for (int qq = 0; qq < 4; ++qq) tot += sspart[wv][m + 16 * qq] + sspart[wv][m + 8 + 16 * qq];
    scale = 1.0f / sqrtf(tot / (float)K + eps);
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int n = (blockIdx.x * RT + rt) * 8 + nrow;
    float now = 0.f;  // the cell's new value
    if (mine && m < M && n < N) {
      float sum = 0.f;
#pragma unroll
      for (int wv = 0; wv < WAVES; ++wv) sum += part[wv][rt][l][e] + part[wv][rt][l + 40][e];  // cell (n + 8, m + 8)
      now = EPI == EPI_ACCUMULATE ? old[rt] + sum * scale : sum * scale;
      c[(size_t)m * ldc + n] = (CT)now;
      if (emits) extra.emit_h[(size_t)m * extra.emit_ldh + n] = (bf16)(emit_g[rt] * now);
    }
    if (emits && mine) squares[rt][m][nrow] = now * now;
  }
  if (!emits) return;
  __syncthreads();  // the waves that are still here
  if (mine && nrow == 0) {
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      float tot = 0.f;
#pragma unroll
      for (int j = 0; j < 8; ++j) tot += squares[rt][m][j];
      extra.emit_ss[(size_t)(blockIdx.x * RT + rt) * 8 + m] = tot;
    }
  }
}

template <int EPI, bool RMS, typename CT>
int launch_fold(const void* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, const void* gamma,
                int gamma_f32, float eps, const NormExtras& extra, hipStream_t stream) {
  const int tiles = (N + 7) / 8, blocks = (K + 127) / 128;  // 128-wide k blocks
  const int waves = blocks >= 16 ? 16 : 4;  // (eight blocks on sixteen waves were measured no faster than on four)
  const int rt = tiles >= 512 ? 2 : 1;
  const int iters = (blocks + waves - 1) / waves >= 2 ? 2 : 1;  // four loads in flight a wave were measured no faster
#define GB_CFG(WV, IT, RT)                                                                                                \
  if (waves == WV && iters == IT && rt == RT)                                                                             \
    hipLaunchKernelGGL((gemm_fold_kernel<WV, IT, RT, EPI, RMS, CT>), dim3((tiles + RT - 1) / RT), dim3(WV * 64), 0, stream, \
                       a, lda, w, ldw, c, ldc, M, N, K, gamma, gamma_f32, eps, extra);
  GB_CFG(4, 1, 1) GB_CFG(4, 1, 2) GB_CFG(4, 2, 1) GB_CFG(4, 2, 2)
  GB_CFG(16, 1, 1) GB_CFG(16, 1, 2) GB_CFG(16, 2, 1) GB_CFG(16, 2, 2)
#undef GB_CFG
  return launched("gemm_bf16 (folded)");
}

// Waves per workgroup, loads in flight per wave and row tiles per workgroup.
inline void skinny_plan(int tiles, int K, int mt, int* waves, int* iters, int* rt) {
  // measured on SmolLM2-1.7B and Llama-3-8B shapes: sixteen waves a workgroup keep the most loads in
  // flight; two row tiles a workgroup halve the re-reading of A once that still leaves workgroups for
  // three quarters of the compute units (384 tiles: better with two; 256 tiles: better with one)
  const int blocks = (K + 63) / 64;               // 64-wide k blocks
  // A wave's k blocks come one after the other, each a round trip to memory: from twelve blocks on sixteen waves take
  // one or two each (a k of 960, fifteen blocks: a decode step of SmolLM2-360M 4 to 8 % faster than with four waves)
  *waves = blocks >= 12 ? 16 : 4;
  *rt = tiles >= 384 ? 2 : 1;
  const int per_wave = (blocks + *waves - 1) / *waves;
  *iters = (mt == 1 && per_wave >= 2) ? 2 : 1;
}

template <int MT, int EPI, bool RMS, typename CT>
int launch_skinny_mt(int tiles, const void* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K,
                     const void* gamma, int gamma_f32, float eps, const NormExtras& extra, const RopeExtras& rope,
                     hipStream_t stream) {
  int waves, iters, rt;
  skinny_plan(tiles, K, MT, &waves, &iters, &rt);
  if constexpr ((EPI == EPI_STORE || EPI == EPI_ACCUMULATE) && !RMS) {
    // Few rows of W (a narrow model's O and down projections, beyond the 8 rows of A that the folded kernel takes):
    // workgroups of 8 rows of W, half of each tile left empty, so that twice as many compute units draw on memory.
    if (tiles < 256 && extra.parts == nullptr) {
      const int halves = (N + 7) / 8;
#define GB_HALF(WV, IT)                                                                                                    \
  if (waves == WV && iters == (IT))                                                                                        \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, WV, (IT), 1, EPI, RMS, CT, true>), dim3(halves), dim3(WV * 64), 0, stream, a, \
                       lda, w, ldw, c, ldc, M, N, K, gamma, gamma_f32, eps, extra, rope);
      GB_HALF(4, 1) GB_HALF(16, 1)
      if (MT == 1) { GB_HALF(4, MT == 1 ? 2 : 1) GB_HALF(16, MT == 1 ? 2 : 1) }
#undef GB_HALF
      return launched("gemm_bf16 (skinny, half tiles)");
    }
  }
  // the rotating product with two tiles a workgroup: a tile and a half each where that divides evenly (three_halves_tile)
  RopeExtras rp = rope;
  rp.three_halves = (EPI == EPI_ROPE && rt == 2 && tiles % 3 == 0) ? 1 : 0;
  const int groups = rp.three_halves ? 2 * tiles / 3 : (tiles + rt - 1) / rt;
#define GB_CFG(WV, IT, RT)                                                                                                 \
  if (waves == WV && iters == (IT) && rt == RT)                                                                            \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, WV, (IT), RT, EPI, RMS, CT>), dim3(groups), dim3(WV * 64), 0, stream, a, lda, \
                       w, ldw, c, ldc, M, N, K, gamma, gamma_f32, eps, extra, rp);
  // the configurations skinny_plan can ask for: two loads in flight only with one column block
  GB_CFG(4, 1, 1) GB_CFG(4, 1, 2) GB_CFG(16, 1, 1) GB_CFG(16, 1, 2)
  if (MT == 1) {
    GB_CFG(4, MT == 1 ? 2 : 1, 1) GB_CFG(4, MT == 1 ? 2 : 1, 2) GB_CFG(16, MT == 1 ? 2 : 1, 1) GB_CFG(16, MT == 1 ? 2 : 1, 2)
  }
#undef GB_CFG
  return launched("gemm_bf16 (skinny)");
}

template <int EPI, bool RMS, typename CT>
int launch_skinny(const void* a, int lda, const bf16* w, int ldw, CT* c, int ldc, int M, int N, int K, const void* gamma,
                  int gamma_f32, float eps, const NormExtras& extra, hipStream_t stream, const RopeExtras& rope = RopeExtras{}) {
  const int tiles = EPI == EPI_SILU_MUL ? (N / 2 + 7) / 8 : (N + 15) / 16;  // EPI_ROPE: N is a multiple of 16
  const int mt = (M + 15) / 16;
#define GB_MT(T) \
  if (mt == T) return launch_skinny_mt<T, EPI, RMS, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, gamma, gamma_f32, eps, extra, rope, stream);
  GB_MT(1) GB_MT(2) GB_MT(3)
#undef GB_MT
  return launch_skinny_mt<4, EPI, RMS, CT>(tiles, a, lda, w, ldw, c, ldc, M, N, K, gamma, gamma_f32, eps, extra, rope, stream);
}

}  // namespace

// epilogue: 0 store, 1 accumulate (float32 C), 2 SiLU-multiply of stacked gate/up rows (C is [M, N/2]).
// gamma != nullptr (at most 64 rows, bfloat16 C, epilogue 0 or 2): a is the float32 residual and the
// product is that of its RMS-normed rows: bf16(gamma * x) as the operand, 1/sqrt(mean(x^2) + eps) on
// the result.
// split_ws != nullptr: a workspace of split_ws_floats floats that the product may use to divide k over
// workgroups (gb_gemm_bf16_split_floats says how many it needs; fewer than that is an error).
// emit_h != nullptr (accumulating product that gb_gemm_bf16_emit_parts accepts): the next norm's operand and
// partial sums are written beside the residual, see NormExtras.  parts != nullptr (at most 64 rows, no
// gamma): the rows of a are such an operand and the product is scaled by the norm's factor from n_parts
// partial sums; eps is that norm's.
extern "C" int gb_gemm_bf16_emit_parts(int M, int N) { return emit_parts(M, N); }
// 0, 1 or 2: see emit_mode.  With 2, gb_gemm_bf16 takes emit_gamma, emit_h and eps (no emit_ss) together with the
// workspace and writes the normed rows to emit_h.
extern "C" int gb_gemm_bf16_emit_mode(int M, int N, int K) { return emit_mode(M, N, K); }

// Floats of workspace with which gb_gemm_bf16 would split k for this product (0: it would not).
extern "C" long long gb_gemm_bf16_split_floats(int M, int N, int K) {
  return M > 16 ? (long long)split_plan(M, N, K).floats : 0;
}

extern "C" int gb_gemm_bf16(const void* a, int lda, const void* w, int ldw, void* c, int ldc, int c_dtype, int M, int N,
                            int K, int epilogue, const void* gamma, int gamma_dtype, float eps, const void* emit_gamma,
                            int emit_gamma_dtype, void* emit_h, int emit_ldh, float* emit_ss, const float* parts, int n_parts,
                            float* split_ws, long long split_ws_floats, hipStream_t stream) {
  GB_REQUIRE(M >= 0 && N > 0 && K > 0, "gemm_bf16: bad sizes M=%d N=%d K=%d", M, N, K);
  GB_REQUIRE(K % 8 == 0, "gemm_bf16: the inner size K=%d must be a multiple of 8 (16-byte operand loads)", K);
  GB_REQUIRE(ldw % 8 == 0 && lda % (gamma ? 4 : 8) == 0, "gemm_bf16: row strides (%d, %d) must keep rows 16-byte aligned", lda, ldw);
  GB_REQUIRE(epilogue >= 0 && epilogue <= 2, "gemm_bf16: unknown epilogue %d", epilogue);
  const int ncols = epilogue == EPI_SILU_MUL ? N / 2 : N;
  GB_REQUIRE(epilogue != EPI_SILU_MUL || N % 2 == 0, "gemm_bf16: stacked gate/up rows need an even N, got %d", N);
  GB_REQUIRE(lda >= K && ldw >= K && ldc >= ncols, "gemm_bf16: a leading dimension is shorter than its row");
  GB_REQUIRE(((uintptr_t)a % 16 == 0) && ((uintptr_t)w % 16 == 0), "gemm_bf16: operands must be 16-byte aligned");
  GB_REQUIRE(epilogue != EPI_ACCUMULATE || c_dtype == kF32, "gemm_bf16: accumulation is into a float32 result");
  GB_REQUIRE(c_dtype == kF32 || c_dtype == kBF16, "gemm_bf16: unknown result dtype %d", c_dtype);
  GB_REQUIRE(!gamma || (M <= 64 && c_dtype == kBF16 && epilogue != EPI_ACCUMULATE && ((uintptr_t)gamma % 16 == 0) &&
                        (gamma_dtype == kF32 || gamma_dtype == kBF16)),
             "gemm_bf16: the fused RMS norm serves up to 64 rows with a bfloat16 result");
  const int emits = emit_h ? emit_mode(M, N, K) : 0;
  GB_REQUIRE(!emit_h || (epilogue == EPI_ACCUMULATE && emit_gamma && emit_ldh >= N && ((uintptr_t)emit_gamma % 16 == 0) &&
                         (emit_gamma_dtype == kF32 || emit_gamma_dtype == kBF16) &&
                         ((emits == 1 && emit_ss) || (emits == 2 && split_ws && emit_ldh % 4 == 0 && ((uintptr_t)emit_h % 8 == 0)))),
             "gemm_bf16: only an accumulating product that gb_gemm_bf16_emit_mode accepts can prepare the next norm");
  GB_REQUIRE(!parts || (M <= 64 && !gamma && n_parts > 0 && epilogue != EPI_ACCUMULATE),
             "gemm_bf16: partial sums of a norm go with at most 64 rows, no gamma, and a storing epilogue");
  const NormExtras extra{emit_gamma, emit_gamma_dtype == kF32, (bf16*)emit_h, emit_ldh, emit_ss, parts, n_parts};
  if (M == 0) return 0;
  const bf16* W = (const bf16*)w;
  if (split_ws != nullptr && M > 16 && !gamma && (!emit_h || emits == 2) && !parts) {  // more than the skinny kernels' best range
    const SplitPlan plan = split_plan(M, N, K, epilogue == EPI_SILU_MUL);
    if (plan.slices > 1 && (epilogue != EPI_SILU_MUL || N % 16 == 0) && (uintptr_t)split_ws % 16 == 0) {
      GB_REQUIRE((long long)plan.floats <= split_ws_floats, "gemm_bf16: the split-k workspace holds %lld floats, %zu are needed",
                 split_ws_floats, plan.floats);
      const bf16* A = (const bf16*)a;
#define GB_SP(EPI, CT) return launch_split<EPI, CT>(A, lda, W, ldw, (CT*)c, ldc, M, N, K, split_ws, plan, stream)
      if (epilogue == EPI_ACCUMULATE)
        return launch_split<EPI_ACCUMULATE, float>(A, lda, W, ldw, (float*)c, ldc, M, N, K, split_ws, plan, stream, &extra, eps);
      if (epilogue == EPI_SILU_MUL && c_dtype == kBF16) GB_SP(EPI_SILU_MUL, bf16);
      if (epilogue == EPI_SILU_MUL) GB_SP(EPI_SILU_MUL, float);
      if (c_dtype == kF32) GB_SP(EPI_STORE, float);
      GB_SP(EPI_STORE, bf16);
#undef GB_SP
    }
  }
  // The narrow tiles without slices: up to 128 rows wherever they give half the compute units a workgroup (with a
  // long enough k the plan above has divided it instead); up to 256 rows where the wide tiles would be few and k is
  // too short to divide (the products of a narrow model: SmolLM2-360M's gate/up of 256 rows, 16.3 -> 11.2 us).
  const int narrow_tiles = ((ncols + 31) / 32) * ((M + SBM - 1) / SBM), wide_tiles = ((N + 127) / 128) * ((M + 127) / 128);
  const bool narrow_pays = M <= STREAM_MAX_ROWS ? narrow_tiles >= 64
                                               : (M <= 2 * STREAM_MAX_ROWS && epilogue == EPI_SILU_MUL && narrow_tiles >= 64 && wide_tiles < 128 && K < 2048);
  if (M > stream_min_rows(M, N, K, epilogue == EPI_SILU_MUL) && narrow_pays && !gamma && !parts && !emit_h && stream_takes(a, lda, w, ldw, K) &&
      (epilogue != EPI_SILU_MUL || N % 16 == 0) && N < 32768) {
    const bf16* A = (const bf16*)a;
#define GB_ST(EPI, CT) return launch_stream<EPI, CT>(A, lda, W, ldw, (CT*)c, ldc, M, N, K, 0, 1, stream)
    if (epilogue == EPI_ACCUMULATE) GB_ST(EPI_ACCUMULATE, float);
    if (epilogue == EPI_SILU_MUL && c_dtype == kBF16) GB_ST(EPI_SILU_MUL, bf16);
    if (epilogue == EPI_SILU_MUL) GB_ST(EPI_SILU_MUL, float);
    if (c_dtype == kF32) GB_ST(EPI_STORE, float);
    GB_ST(EPI_STORE, bf16);
#undef GB_ST
  }
  // 17 to 64 rows by very many rows of W (the vocabulary product of a large decode batch): measured twice as fast
  // through the tiles below as through the skinny kernel with four column blocks (49,152 x 2,048: 102 -> about 50 us),
  // and with two column blocks as fast or faster (49,152 x 960 at 17 to 32 rows: 30 -> 25 us)
  const bool wide_head = M > 16 && N >= 32768 && !gamma && !parts;
  if (M <= 64 && !wide_head) {
    const int gf = gamma_dtype == kF32;
    if (fold_pays(M, N) && epilogue != EPI_SILU_MUL && !parts) {
      if (gamma) return launch_fold<EPI_STORE, true, bf16>(a, lda, W, ldw, (bf16*)c, ldc, M, N, K, gamma, gf, eps, extra, stream);
      if (epilogue == EPI_ACCUMULATE) return launch_fold<EPI_ACCUMULATE, false, float>(a, lda, W, ldw, (float*)c, ldc, M, N, K, nullptr, 0, 0.f, extra, stream);
      if (c_dtype == kF32) return launch_fold<EPI_STORE, false, float>(a, lda, W, ldw, (float*)c, ldc, M, N, K, nullptr, 0, 0.f, extra, stream);
      return launch_fold<EPI_STORE, false, bf16>(a, lda, W, ldw, (bf16*)c, ldc, M, N, K, nullptr, 0, 0.f, extra, stream);
    }
    if (gamma) {
      if (epilogue == EPI_STORE) return launch_skinny<EPI_STORE, true, bf16>(a, lda, W, ldw, (bf16*)c, ldc, M, N, K, gamma, gf, eps, extra, stream);
      return launch_skinny<EPI_SILU_MUL, true, bf16>(a, lda, W, ldw, (bf16*)c, ldc, M, N, K, gamma, gf, eps, extra, stream);
    }
#define GB_SK(EPI, CT) return launch_skinny<EPI, false, CT>(a, lda, W, ldw, (CT*)c, ldc, M, N, K, nullptr, 0, eps, extra, stream)
    if (epilogue == EPI_STORE && c_dtype == kF32) GB_SK(EPI_STORE, float);
    if (epilogue == EPI_STORE && c_dtype == kBF16) GB_SK(EPI_STORE, bf16);
    if (epilogue == EPI_ACCUMULATE) GB_SK(EPI_ACCUMULATE, float);
    if (epilogue == EPI_SILU_MUL && c_dtype == kF32) GB_SK(EPI_SILU_MUL, float);
    GB_SK(EPI_SILU_MUL, bf16);
#undef GB_SK
  }
  const bf16* A = (const bf16*)a;
  if (ring_pays(epilogue, a, lda, w, ldw, M, N, K) && (epilogue != EPI_SILU_MUL || N % 2 == 0)) {
#define GB_RG(EPI, CT) return launch_ring<EPI, CT>(A, lda, W, ldw, (CT*)c, ldc, M, N, K, stream)
    if (epilogue == EPI_ACCUMULATE) GB_RG(EPI_ACCUMULATE, float);
    if (epilogue == EPI_SILU_MUL && c_dtype == kBF16) GB_RG(EPI_SILU_MUL, bf16);
    if (epilogue == EPI_SILU_MUL) GB_RG(EPI_SILU_MUL, float);
    if (c_dtype == kF32) GB_RG(EPI_STORE, float);
    GB_RG(EPI_STORE, bf16);
#undef GB_RG
  }
#define GB_TL(EPI, CT) return launch_tiled<EPI, CT>(A, lda, W, ldw, (CT*)c, ldc, M, N, K, stream)
  if (epilogue == EPI_ACCUMULATE) GB_TL(EPI_ACCUMULATE, float);
  if (epilogue == EPI_SILU_MUL && c_dtype == kBF16) GB_TL(EPI_SILU_MUL, bf16);
  if (epilogue == EPI_SILU_MUL) GB_TL(EPI_SILU_MUL, float);
  if (c_dtype == kF32) GB_TL(EPI_STORE, float);
  GB_TL(EPI_STORE, bf16);
#undef GB_TL
}

// The QKV product of a step of at most 64 rows with EPI_ROPE (see RopeExtras): c is the stacked rows
// [M][(nh + 2 nkv) hd] (or [M][nh hd] with nkv == 0: queries only), bfloat16.  gamma / parts as in
// gb_gemm_bf16 (the norm before the product).
extern "C" int gb_gemm_bf16_rope(const void* a, int lda, const void* w, int ldw, void* c, int ldc, int M, int N, int K,
                                 const void* gamma, int gamma_dtype, float eps, const float* parts, int n_parts,
                                 const float* cosv, const float* sinv, const int32_t* slots, void* k_pages, void* v_pages,
                                 int nh, int nkv, int hd, int page_size, hipStream_t stream) {
  GB_REQUIRE(M > 0 && M <= 64 && N > 0 && K > 0 && K % 8 == 0, "gemm_bf16_rope: bad sizes M=%d N=%d K=%d (at most 64 rows)", M, N, K);
  GB_REQUIRE(hd >= 16 && hd % 16 == 0 && nh > 0 && nkv >= 0 && N == (nh + 2 * nkv) * hd,
             "gemm_bf16_rope: N=%d is not (nh + 2 nkv) hd with nh=%d nkv=%d hd=%d (a multiple of 16)", N, nh, nkv, hd);
  GB_REQUIRE(ldw % 8 == 0 && lda % (gamma ? 4 : 8) == 0 && lda >= K && ldw >= K && ldc >= N && ((uintptr_t)a % 16 == 0) &&
                 ((uintptr_t)w % 16 == 0),
             "gemm_bf16_rope: operands must be 16-byte aligned rows");
  GB_REQUIRE((cosv == nullptr) == (sinv == nullptr), "gemm_bf16_rope: cos and sin come together");
  GB_REQUIRE(!slots || (k_pages && v_pages && page_size > 0 && nkv > 0), "gemm_bf16_rope: slots given without pages");
  GB_REQUIRE(!gamma || (((uintptr_t)gamma % 16 == 0) && (gamma_dtype == kF32 || gamma_dtype == kBF16) && !parts),
             "gemm_bf16_rope: gamma must be aligned float32 or bfloat16, and not given together with parts");
  GB_REQUIRE(!parts || n_parts > 0, "gemm_bf16_rope: partial sums of a norm without a count");
  const NormExtras extra{nullptr, 0, nullptr, 0, nullptr, parts, n_parts};
  const RopeExtras rope{cosv, sinv, slots, (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, page_size, 0};
  if (gamma)
    return launch_skinny<EPI_ROPE, true, bf16>(a, lda, (const bf16*)w, ldw, (bf16*)c, ldc, M, N, K, gamma, gamma_dtype == kF32,
                                               eps, extra, stream, rope);
  return launch_skinny<EPI_ROPE, false, bf16>(a, lda, (const bf16*)w, ldw, (bf16*)c, ldc, M, N, K, nullptr, 0, eps, extra,
                                              stream, rope);
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_gemm_bf16)
GB_TAPED(gb_gemm_bf16_rope)
