// Paged attention in bfloat16 on the matrix cores, for decoding and for prompt portions.
//
// Per request and kv head the work is out[col] = softmax(q[col] . K^T * scale) . V for "columns"
// that share the keys.  When decoding, the columns are the up to 16 query heads of one token that
// map to the kv head (grouped-query attention reads each key once for the whole group), and the
// inner step over 64 keys is:
//   S^T[key, col] = K[key, :] . Q[col, :]     v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 dims straight
//                                             from the key page (16 bytes a lane), B = the query columns
//   running max / sum per column in 32-bit, keys outside [lo, hi] of the column masked to -inf
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col]   A = 16 dims x 32 keys from the transposed value
//                                             page (8 bytes a lane from each of two tiles), B = the
//                                             probabilities, taken from the score registers as they
//                                             are (the k order of both operands is permuted alike)
// so neither scores nor probabilities pass through LDS, and keys and values go from memory into
// MFMA operands directly.  Pages: keys [page][kv head][hd / 8][slot][8], values [page][kv head][hd][slot].
// A prompt portion's columns are 32 or 64 consecutive tokens of one query head, with the same
// scheme on the 32x32x16 instruction (described at its kernel).
//
// Decoding splits a request's context into chunks of a multiple of 256 keys, one workgroup per
// (chunk, kv head, request), four waves taking 64 keys each in turn; partial results are merged
// in a fixed order (waves in LDS, chunks by a second kernel), so the result is the same on every
// run.  crates/glassbox-core/src/model.rs:285-312 is the formula.
#include "attention_bf16.h"
#include "common.h"

#include <mutex>

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
// read once and not again in this kernel: the caches need not keep it
__device__ __forceinline__ bf16x8 load8_once(const bf16* p) { return __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p)); }
__device__ __forceinline__ bf16x4 load4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }
__device__ __forceinline__ bf16x4 load4_once(const bf16* p) { return __builtin_nontemporal_load(reinterpret_cast<const bf16x4*>(p)); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (bf16)0.f;
  return z;
}

template <int HD>
struct Running {
  float m, l;  // running maximum; this lane's share of the running sum
  f32x4 acc[HD / 16];
};

template <int HD>
__device__ __forceinline__ void reset(Running<HD>& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int b = 0; b < HD / 16; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) st.acc[b][r] = 0.f;
}

// 64 keys from kbase (a multiple of 16).  Lane (col = lane % 16, c = lane / 16).  Keys in
// [lo, hi] count for this lane's column; [clamp_lo, clamp_hi] (the same for the whole wave) is a
// range of keys known to have pages: tiles outside it are redirected to a tile inside it, and all
// their keys are masked anyway.
template <int HD>
__device__ __forceinline__ void attend64(Running<HD>& st, const bf16x8* qf, const bf16* __restrict__ kp,
                                         const bf16* __restrict__ vp, const int32_t* __restrict__ table, int nkv, int kvh,
                                         int P, int kbase, int lo, int hi, int clamp_lo, int clamp_hi, float scale,
                                         int lane) {
  constexpr int KS = (HD + 31) / 32, DB = HD / 16;
  const int j = lane & 15, c = lane >> 4;
  bf16x8 kf[4][KS];
  bf16x4 vf[DB][4];
  const int tlo = clamp_lo & ~15, thi = clamp_hi & ~15;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    const int kt = kbase + 16 * t;
    const int kc = min(max(kt, tlo), thi);
    const int page = table[kc / P];
    const int slot0 = kc % P;
    // pieces of 8 dimensions, of each the page's slots side by side (key_piece()): the 16 lanes of a group read 256 bytes
    const bf16* kb = kp + ((size_t)page * nkv + kvh) * P * HD + (slot0 + j) * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + c * 8;
      kf[t][ks] = d0 < HD ? load8_once(kb + (size_t)(ks * 4 + c) * P * 8) : zero8();
    }
    const bf16* vb = vp + ((size_t)page * nkv + kvh) * HD * P + slot0 + 4 * c;
#pragma unroll
    for (int b = 0; b < DB; ++b) vf[b][t] = load4_once(vb + (size_t)(16 * b + j) * P);
  }
  float s[4][4];
  float mx = -INFINITY;
#pragma unroll
  for (int t = 0; t < 4; ++t) {
    f32x4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) a = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kf[t][ks], qf[ks], a, 0, 0, 0);
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int key = kbase + 16 * t + 4 * c + r;
      s[t][r] = (key >= lo && key <= hi) ? a[r] * scale : -INFINITY;
      mx = fmaxf(mx, s[t][r]);
    }
  }
  mx = fmaxf(mx, __shfl_xor(mx, 16, kWave));
  mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
  const float m_new = fmaxf(st.m, mx);
  const float alpha = st.m == -INFINITY ? 0.f : __expf(st.m - m_new);
  float sum = 0.f;
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      s[t][r] = s[t][r] == -INFINITY ? 0.f : __expf(s[t][r] - m_new);
      sum += s[t][r];
    }
  st.l = st.l * alpha + sum;
  st.m = m_new;
#pragma unroll
  for (int b = 0; b < DB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) st.acc[b][r] *= alpha;
#pragma unroll
  for (int u = 0; u < 2; ++u) {
    bf16x8 pf;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      pf[r] = (bf16)s[2 * u][r];
      pf[4 + r] = (bf16)s[2 * u + 1][r];
    }
#pragma unroll
    for (int b = 0; b < DB; ++b) {
      bf16x8 af;
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        af[r] = vf[b][2 * u][r];
        af[4 + r] = vf[b][2 * u + 1][r];
      }
      st.acc[b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af, pf, st.acc[b], 0, 0, 0);
    }
  }
}

// ----------------------------------------------------------------------------- decode
// grid (chunks, kv heads, requests); request s is row s of q and out, at position positions[s].
// WAVES waves take 64 keys each in turn; dynamic LDS holds their partial results for the merge:
// WAVES * (32 + HD * G) floats, G the query heads per kv head.
template <int HD, int WAVES>
__global__ __launch_bounds__(WAVES * 64) void decode_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                                            int out_stride, float* __restrict__ ws_acc,
                                                            float* __restrict__ ws_ml, const int32_t* __restrict__ positions,
                                                            const int32_t* __restrict__ tables, int table_stride,
                                                            const bf16* __restrict__ kp, const bf16* __restrict__ vp, int nh,
                                                            int nkv, int P, float scale, int window, int chunk, int splits) {
  constexpr int KS = (HD + 31) / 32, DB = HD / 16;
  extern __shared__ float decode_lds[];
  const int s = blockIdx.z, kvh = blockIdx.y, split = blockIdx.x;
  const int G = nh / nkv;
  float* sm_m = decode_lds;               // [WAVES][16]
  float* sm_l = sm_m + WAVES * 16;        // [WAVES][16]
  float* sm_acc = sm_l + WAVES * 16;      // [WAVES][HD][G]
  const int pos = positions[s];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int c0 = split * chunk;
  if (c0 > pos || c0 + chunk <= lo) return;  // this chunk holds no key of the request
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int col = lane & 15;
  const int32_t* table = tables + (size_t)s * table_stride;

  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + (lane >> 4) * 8;
    qf[ks] = (col < G && d0 < HD) ? load8(q + (size_t)s * q_stride + (size_t)(kvh * G + col) * HD + d0) : zero8();
  }
  Running<HD> st;
  reset(st);
  const int col_lo = col < G ? lo : 1, col_hi = col < G ? pos : 0;
  const int end = min(c0 + chunk, pos + 1);
  for (int kb = c0 + wave * 64; kb < end; kb += 64 * WAVES) {
    if (kb + 64 <= lo) continue;
    attend64<HD>(st, qf, kp, vp, table, nkv, kvh, P, kb, col_lo, col_hi, lo, pos, scale, lane);
  }
  st.l += __shfl_xor(st.l, 16, kWave);
  st.l += __shfl_xor(st.l, 32, kWave);
  if (lane < 16) {
    sm_m[wave * 16 + col] = st.m;
    sm_l[wave * 16 + col] = st.l;
  }
  if (col < G) {
#pragma unroll
    for (int b = 0; b < DB; ++b)
#pragma unroll
      for (int r = 0; r < 4; ++r) sm_acc[((size_t)wave * HD + 16 * b + 4 * (lane >> 4) + r) * G + col] = st.acc[b][r];
  }
  __syncthreads();
  // the waves' partial results, combined in wave order
  for (int cell = tid; cell < HD * G; cell += WAVES * 64) {
    const int d = cell / G, cc = cell % G;
    float M = sm_m[cc];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) M = fmaxf(M, sm_m[w * 16 + cc]);
    float val = 0.f, L = 0.f;
#pragma unroll
    for (int w = 0; w < WAVES; ++w) {
      const float mw = sm_m[w * 16 + cc];
      const float f = mw == -INFINITY ? 0.f : __expf(mw - M);
      val += sm_acc[((size_t)w * HD + d) * G + cc] * f;
      L += sm_l[w * 16 + cc] * f;
    }
    const int head = kvh * G + cc;
    if (splits == 1) {
      out[(size_t)s * out_stride + (size_t)head * HD + d] = (bf16)(val / L);
    } else {
      const size_t slot = ((size_t)s * nh + head) * splits + split;
      ws_acc[slot * HD + d] = val;
      if (d == 0) {
        ws_ml[slot * 2] = M;
        ws_ml[slot * 2 + 1] = L;
      }
    }
  }
}

// One block of 256 threads per (request, head): the chunks' partial results, combined in a fixed order.
// The chunks are dealt to 256 / hd groups of threads, each thread of a group taking one dimension; the groups' sums
// meet in LDS.  Everything a thread reads from memory depends on nothing but the request's position, so it is all
// asked for at once (a chunk's maximum and sum by thread k, the first partial results of the thread's dimension),
// and the maximum over the chunks and the sum of their weights are taken wave by wave, not by one thread in turn:
// the kernel is short, and round trips and serial loops are what it consists of.
__global__ __launch_bounds__(256) void decode_reduce_kernel(const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                                                            bf16* __restrict__ out, int out_stride,
                                                            const int32_t* __restrict__ positions, int nh, int hd, int window,
                                                            int chunk, int splits) {
  constexpr int EARLY = 4;           // partial results a thread asks for before it knows their weights
  __shared__ float sm_f[256];        // chunk k's weight exp(m_k - M)
  __shared__ float sm_part[256];     // [group][dimension]
  __shared__ float sm_top[4], sm_sum[4];
  const int s = blockIdx.x / nh, head = blockIdx.x % nh, tid = threadIdx.x, lane = tid % 64, wave = tid / 64;
  const int pos = positions[s];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int first = lo / chunk, last = pos / chunk, count = last - first + 1;  // at most 256 chunks hold keys
  const size_t base = ((size_t)s * nh + head) * splits + first;
  const int groups = 256 / hd;  // hd <= 128: at least two
  const int d = tid % hd, group = tid / hd;
  float mine = -INFINITY, mine_l = 0.f, early[EARLY];
  if (tid < count) {
    mine = ws_ml[(base + tid) * 2];
    mine_l = ws_ml[(base + tid) * 2 + 1];
  }
#pragma unroll
  for (int i = 0; i < EARLY; ++i) {
    const int k = group + i * groups;
    early[i] = (group < groups && k < count) ? ws_acc[(base + k) * hd + d] : 0.f;
  }
  float top = mine;
#pragma unroll
  for (int off = 32; off >= 1; off >>= 1) top = fmaxf(top, __shfl_xor(top, off, kWave));
  if (lane == 0) sm_top[wave] = top;
  __syncthreads();
  top = fmaxf(fmaxf(sm_top[0], sm_top[1]), fmaxf(sm_top[2], sm_top[3]));
  const float f = tid < count ? __expf(mine - top) : 0.f;
  sm_f[tid] = f;
  float sum = f * mine_l;  // the chunks' sums, weighted: added lane pairs first, then the waves in order
#pragma unroll
  for (int off = 1; off <= 32; off <<= 1) sum += __shfl_xor(sum, off, kWave);
  if (lane == 0) sm_sum[wave] = sum;
  __syncthreads();
  float val = 0.f;
  if (group < groups) {
#pragma unroll
    for (int i = 0; i < EARLY; ++i) {
      const int k = group + i * groups;
      if (k < count) val += early[i] * sm_f[k];
    }
    for (int k = group + EARLY * groups; k < count; k += groups) val += ws_acc[(base + k) * hd + d] * sm_f[k];
  }
  sm_part[tid] = val;
  __syncthreads();
  if (tid < hd) {
    float total = 0.f;
    for (int g = 0; g < groups; ++g) total += sm_part[g * hd + tid];
    const float l = ((sm_sum[0] + sm_sum[1]) + sm_sum[2]) + sm_sum[3];
    out[(size_t)s * out_stride + (size_t)head * hd + tid] = (bf16)(total / l);
  }
}

// ---------------------------------------------------------------------------- prefill
// A wave takes blocks of 32 consecutive tokens of one query head; v_mfma_f32_32x32x16_bf16 throughout.
// Per 64 keys:
//   S^T[key, tok]   A = 32 keys x 16 dims (lane: row lane%32, dims 8*(lane/32)..+7 of the k-step),
//                   B = the query tokens alike; the result lane holds token lane%32 and rows
//                   8*(r/4) + 4*(lane/32) + r%4 of the 32-row tile
//   O^T[dim, tok]   A = 32 dims x 16 keys from the transposed value page, B = probabilities: registers
//                   8h..8h+7 of a score tile are, as they stand, the B operand of the k-step over rows
//                   16h..16h+15, lane group g holding rows 4g..4g+3 and 8+4g..8+4g+3 of them
// Which key a row of the score tile stands for is free: within each group of 16 rows the keys are
// dealt so that those eight rows of a lane group are the neighbouring keys 8g..8g+7.  The value
// operand of a lane is then one 16-byte word of its dimension's row in the page, and a load
// instruction of the wave reads whole 32-byte rows (the cache serves 64 bytes at a time; half-used
// pieces were what bounded this kernel).
// Scores stay raw in the registers; softmax works on exp2(raw*c - max*c) with c = scale*log2(e).
// Causal work grows with the position, so a wave takes block i and block n-1-i of its request's
// portion: every wave then has the same number of (token, key) pairs.  With QB == 2 both blocks are
// live at once and share the key and value fragments where their key ranges overlap (ACT says
// which are live in a step); with QB == 1 (head sizes whose accumulators leave no room) one after
// the other.
// Where a wave's key and value fragments come from.  Everything here is the same for all lanes of a
// wave, so page lookups and page addresses are scalar work.
struct PageSource {
  const bf16* __restrict__ kp;
  const bf16* __restrict__ vp;
  const int32_t* __restrict__ table;
  int nkv, kvh, shift;  // pages of 1 << shift keys
  int tlo, thi;         // groups of 16 keys outside [tlo, thi] are redirected into it (their keys are masked anyway)
  // offset, in elements of a page array of one kv head, of the page and slot that hold key k
  __device__ __forceinline__ size_t page_of(int k, int* slot) const {
    const int kc = min(max(k, tlo), thi);
    *slot = kc & ((1 << shift) - 1);
    return ((size_t)table[kc >> shift] * nkv + kvh);
  }
};

template <int HD, int T>
__device__ __forceinline__ void load_keys(bf16x8 (&kf)[T][HD / 16], const PageSource& src, int kbase, int lane) {
  const int col = lane & 31, g = lane >> 5;
  // row r of a group of 16 rows of the score tile takes key 8*((r>>2)&1) + 4*(r>>3) + (r&3) of the group:
  // the probabilities a lane then holds for a value product are those of 8 neighbouring keys
  const int r16 = col & 15, key16 = ((r16 >> 2) & 1) * 8 + (r16 >> 3) * 4 + (r16 & 3);
  // a key's dimensions lie in pieces of 8, of each piece the page's slots side by side (key_piece()): this lane's
  // piece of MFMA step ks is number 2 ks + g, and the lanes of a group of 16 keys read 256 bytes in a row
  const int mine = ((g << src.shift) + key16) * 8;
#pragma unroll
  for (int t = 0; t < T; ++t) {
    int s0, s1;  // a tile of 32 keys is two groups of 16, each within one page
    const size_t p0 = src.page_of(kbase + 32 * t, &s0), p1 = src.page_of(kbase + 32 * t + 16, &s1);
    const bf16* b0 = src.kp + (p0 << src.shift) * HD + s0 * 8;
    const bf16* b1 = src.kp + (p1 << src.shift) * HD + s1 * 8;
    const bf16* kb = ((col & 16) ? b1 : b0) + mine;
#pragma unroll
    for (int ks = 0; ks < HD / 16; ++ks) kf[t][ks] = load8(kb + ((size_t)(16 * ks) << src.shift));
  }
}

template <int HD, int T>
__device__ __forceinline__ void load_values(bf16x8 (&vf)[(HD + 31) / 32][2 * T], const PageSource& src, int kbase, int lane) {
  const int col = lane & 31, g = lane >> 5;
  const int mine = (col << src.shift) + 8 * g;
#pragma unroll
  for (int u = 0; u < 2 * T; ++u) {
    int slot;
    const size_t pg = src.page_of(kbase + 16 * u, &slot);
    const bf16* vb = src.vp + ((pg * HD) << src.shift) + slot + mine;
#pragma unroll
    for (int b = 0; b < (HD + 31) / 32; ++b)
      vf[b][u] = (32 * b + 32 <= HD || 32 * b + col < HD) ? load8(vb + ((size_t)(32 * b) << src.shift)) : zero8();
  }
}

// One step over the 32 T keys from kbase (T = 2; T = 1 for the head sizes whose fragments of 64 keys do not
// fit the registers), whose fragments kf and vf hold.  The live blocks take their
// turn one after the other (scores, softmax, values), so that only one block's scores are in
// registers at a time; as soon as the last block's score products have read kf it is loaded again
// for the keys from `next`, and vf likewise after the last value products, so that those loads are
// in flight during the arithmetic in between.
template <int HD, int QB, int ACT, int T = 2>
__device__ __forceinline__ void attend64_q32(float (&m)[QB], float (&l)[QB], f32x16 (&acc)[QB][(HD + 31) / 32],
                                             const bf16x8* __restrict__ q_lds, int q_at, bf16x8 (&kf)[T][HD / 16],
                                             bf16x8 (&vf)[(HD + 31) / 32][2 * T], const PageSource& src, int kbase, int next,
                                             const int (&lo)[QB], const int (&hi)[QB], bool mask, float c, int lane) {
  constexpr int KS = HD / 16, DB = (HD + 31) / 32;
  constexpr int LAST = (ACT & 2) ? 1 : 0;
  const int g = lane >> 5;
  // the compiler must not know that the query fragments are the same in every step, or it reads them
  // once before the loop and has no registers to keep them in
  asm volatile("" : "+v"(q_at));
  const bf16x8* qf = q_lds + q_at;
#pragma unroll
  for (int qb = 0; qb < QB; ++qb) {
    if (!((ACT >> qb) & 1)) continue;
    f32x16 s[T];
#pragma unroll
    for (int t = 0; t < T; ++t) {
#pragma unroll
      for (int r = 0; r < 16; ++r) s[t][r] = 0.f;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        s[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[t][ks], qf[(qb * KS + ks) * 64], s[t], 0, 0, 0);
    }
    if (qb == LAST) {
      // not earlier: above the score products the old and the new fragments would both need registers
      __builtin_amdgcn_sched_barrier(0);
      load_keys<HD, T>(kf, src, next, lane);
    }
    if (mask) {  // the same for the whole wave
#pragma unroll
      for (int t = 0; t < T; ++t)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int key = kbase + 32 * t + 16 * (r >> 3) + 8 * g + 4 * ((r >> 2) & 1) + (r & 3);
          if (key < lo[qb] || key > hi[qb]) s[t][r] = -INFINITY;
        }
    }
    float mx = -INFINITY;
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s[t][r]);
    mx = fmaxf(mx, __shfl_xor(mx, 32, kWave));
    const float m_new = fmaxf(m[qb], mx);
    const float m_ref = m_new == -INFINITY ? 0.f : m_new;  // a column with no key yet
    const float alpha = m[qb] == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m[qb] - m_ref) * c);
    const float mc = m_ref * c;
    float sum = 0.f;
#pragma unroll
    for (int t = 0; t < T; ++t)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        s[t][r] = __builtin_amdgcn_exp2f(fmaf(s[t][r], c, -mc));
        sum += s[t][r];
      }
    l[qb] = l[qb] * alpha + sum;
    m[qb] = m_new;
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[qb][b][r] *= alpha;
    }
#pragma unroll
    for (int u = 0; u < 2 * T; ++u) {
      bf16x8 pf;
#pragma unroll
      for (int e = 0; e < 8; ++e) pf[e] = (bf16)s[u >> 1][8 * (u & 1) + e];
#pragma unroll
      for (int b = 0; b < DB; ++b) acc[qb][b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[b][u], pf, acc[qb][b], 0, 0, 0);
    }
  }
  __builtin_amdgcn_sched_barrier(0);
  load_values<HD, T>(vf, src, next, lane);
}

// What a wave knows of one block of 32 tokens: the keys [first, last] that any of its tokens sees, and
// the keys [free_lo, free_hi] that all of them see (no mask needed there, if the block is whole).
struct BlockRange {
  int first, last, free_lo, free_hi;
  bool whole;
  // of the keys kb .. kb + span - 1
  __device__ bool unmasked(int kb, int span = 64) const { return whole && kb >= free_lo && kb + span - 1 <= free_hi; }
};

__device__ __forceinline__ BlockRange block_range(int t0, int qlen, int p0, int window) {
  BlockRange r;
  const int t1 = min(t0 + 32, qlen) - 1;
  r.whole = t0 + 32 <= qlen;
  r.last = p0 + t1;
  r.first = window > 0 ? max(0, p0 + t0 - window + 1) : 0;
  r.free_hi = p0 + t0;
  r.free_lo = window > 0 ? max(0, p0 + t1 - window + 1) : 0;
  return r;
}

template <int HD>
__device__ __forceinline__ void store_block(const f32x16 (&acc)[(HD + 31) / 32], float l, bf16* __restrict__ orow, int g) {
  const float inv = 1.0f / l;
#pragma unroll
  for (int b = 0; b < (HD + 31) / 32; ++b)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int d0 = 32 * b + 8 * jj + 4 * g;
      if (32 * b + 32 <= HD || d0 < HD) {
        bf16x4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = (bf16)(acc[b][4 * jj + r] * inv);
        *reinterpret_cast<bf16x4*>(orow + d0) = o;
      }
    }
}

// A block's sums as they stand (not divided by l), for the pass that adds the parts of workgroups that shared its
// keys: part_acc [part][row][head][HD], part_ml [part][row][head][2] = the maximum and l.
template <int HD>
__device__ __forceinline__ void store_part(const f32x16 (&acc)[(HD + 31) / 32], float m, float l, float* __restrict__ acc_row,
                                           float* __restrict__ ml, int g) {
#pragma unroll
  for (int b = 0; b < (HD + 31) / 32; ++b)
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int d0 = 32 * b + 8 * jj + 4 * g;
      if (32 * b + 32 <= HD || d0 < HD) {
        f32x4 o;
#pragma unroll
        for (int r = 0; r < 4; ++r) o[r] = acc[b][4 * jj + r];
        *reinterpret_cast<f32x4*>(acc_row + d0) = o;
      }
    }
  if (g == 0) {
    ml[0] = m;
    ml[1] = l;
  }
}

// Adds the parts in their order: one workgroup of HD threads per (row, head).
__global__ void prefill_parts_kernel(const float* __restrict__ part_acc, const float* __restrict__ part_ml, bf16* __restrict__ out,
                                     int out_stride, int first_row, int n_rows, int nh, int hd, int parts, float c) {
  const int row = blockIdx.x / nh, head = blockIdx.x % nh, d = threadIdx.x;
  if (d >= hd) return;
  const size_t cell = (size_t)row * nh + head, stride = (size_t)n_rows * nh;
  float top = -INFINITY;
  for (int k = 0; k < parts; ++k) top = fmaxf(top, part_ml[(k * stride + cell) * 2]);
  float val = 0.f, l = 0.f;
  for (int k = 0; k < parts; ++k) {
    const float mk = part_ml[(k * stride + cell) * 2];
    const float f = mk == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((mk - top) * c);
    val += part_acc[(k * stride + cell) * hd + d] * f;
    l += part_ml[(k * stride + cell) * 2 + 1] * f;
  }
  out[(size_t)(first_row + row) * out_stride + (size_t)head * hd + d] = (bf16)(val / l);
}

// The waves of a group that shared a block's keys add up their maxima, sums and accumulators into wave 0 through LDS,
// pair by pair: in round one wave 1 hands over to wave 0, 3 to 2, 5 to 4 ...; in round two wave 2 to wave 0, 6 to 4; and
// so on, so that eight waves need three rounds and not seven (`handed`: SPLIT/2 places of DB*16*64 floats, `handed_ml`:
// SPLIT/2 x 2*64, both the group's own).  The order of the additions is fixed by the wave numbers.  Every wave of the
// workgroup calls this (it holds barriers); `again` is false only at the workgroup's first call.
template <int DB, int SPLIT>
__device__ __forceinline__ void hand_over(float& m, float& l, f32x16 (&acc)[DB], float* handed, float* handed_ml, int half,
                                          int lane, float c, bool again) {
  static_assert((SPLIT & (SPLIT - 1)) == 0, "waves pair up round by round");
#pragma unroll
  for (int step = 1; step < SPLIT; step *= 2) {
    if (again || step > 1) __syncthreads();  // what was handed over before has been taken
    const int place = half / (2 * step);
    float* there = handed + (size_t)place * (DB * 16 * 64);
    float* there_ml = handed_ml + place * 128;
    if ((half & (2 * step - 1)) == step) {
      there_ml[lane] = m;
      there_ml[64 + lane] = l;
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) there[(b * 16 + r) * 64 + lane] = acc[b][r];
    }
    __syncthreads();
    if ((half & (2 * step - 1)) == 0) {
      const float m1 = there_ml[lane], l1 = there_ml[64 + lane];
      const float top = fmaxf(m, m1);
      const float ref = top == -INFINITY ? 0.f : top;
      const float a0 = m == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m - ref) * c);
      const float a1 = m1 == -INFINITY ? 0.f : __builtin_amdgcn_exp2f((m1 - ref) * c);
      m = top;
      l = l * a0 + l1 * a1;
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[b][r] = acc[b][r] * a0 + there[(b * 16 + r) * 64 + lane] * a1;
    }
  }
}

// grid (groups of PAIRS pairs of blocks, query heads, requests from seq_base on); pair w of a request is its
// blocks w and n-1-w of 32 tokens.  SPLIT waves share a pair: they take its tiles of 64 keys in turn, and at the
// end the others hand their sums to the first through LDS.  One wave a pair is best when the pairs alone give
// every SIMD a wave; short portions and few heads do not, and then the keys are what is left to divide.
template <int HD, int QB, int PAIRS, int SPLIT>
__global__ __launch_bounds__(64 * PAIRS * SPLIT, 2) void prefill_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                                      int out_stride, const int32_t* __restrict__ q_start,
                                                      const int32_t* __restrict__ q_len, const int32_t* __restrict__ pos0,
                                                      int seq_base, const int32_t* __restrict__ tables, int table_stride,
                                                      const bf16* __restrict__ kp, const bf16* __restrict__ vp, int nh, int nkv,
                                                      int page_shift, float scale, int window, float* __restrict__ part_acc,
                                                      float* __restrict__ part_ml, int parts, int first_row, int n_rows) {
  // parts > 1: `parts` workgroups share a group's pairs, taking the tiles of keys in turn like the waves of a pair
  // do; each writes its sums to part_acc / part_ml (rows counted from first_row), and prefill_parts_kernel adds them.
  constexpr int KS = HD / 16, DB = (HD + 31) / 32;
  // Workgroups go to the chip's eight dies in turn, each die with an L2 of its own.  The ones that
  // land on one die are given consecutive units of work, so that a head's keys and values, which all
  // of its token groups read, are fetched into one L2 rather than eight.
  constexpr int kDies = 8;
  const int gx = gridDim.x, gy = gridDim.y, total = gx * gy * gridDim.z;
  const int linear = blockIdx.x + gx * (blockIdx.y + gy * blockIdx.z);
  const int die = linear % kDies;
  const int unit = die * (total / kDies) + min(die, total % kDies) + linear / kDies;
  const int seq = seq_base + unit / (gx * gy), head = unit / gx % gy, group = unit % gx / parts, part = unit % gx % parts;
  static_assert(QB == 2 || PAIRS == 1 || SPLIT == 1, "one block at a time: waves share keys only if the workgroup is one pair");
  static_assert(PAIRS * SPLIT <= 8, "two waves a SIMD have the registers this kernel needs");
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave_of_all = __builtin_amdgcn_readfirstlane(tid >> 6);  // the same in all lanes: what follows from it is scalar
  const int wave = wave_of_all / SPLIT, half = wave_of_all % SPLIT;  // which pair; which of its tiles of keys
  const int qlen = q_len[seq];
  const int blocks = (qlen + 31) / 32;
  const int w = group * PAIRS + wave;
  const bool works = 2 * w < blocks;
  if (SPLIT == 1 && !works) return;
  if (2 * group * PAIRS >= blocks) return;  // the whole workgroup; with SPLIT > 1 every wave left goes to the barriers below
  const int col = lane & 31, g = lane >> 5;
  const int p0 = pos0[seq];
  const int kvh = head / (nh / nkv);
  PageSource src{kp, vp, tables + (size_t)seq * table_stride, nkv, kvh, page_shift, 0, 0};
  const size_t row0 = (size_t)q_start[seq];
  const float c = scale * 1.4426950408889634f;
  constexpr int T = QB == 2 ? 2 : 1;  // tiles of 32 keys a step: with one block live at a time (the larger head
                                      // sizes) the fragments of 64 keys would not fit the registers
  bf16x8 kf[T][KS];
  bf16x8 vf[DB][2 * T];
  // The query fragments wait in LDS, each lane's own in a place of its own (no lane reads another's):
  // they are needed once per step over 64 keys, and the registers are better spent on the accumulators.
  __shared__ bf16x8 q_lds[PAIRS * QB * KS * 64];
  __shared__ float handed[SPLIT > 1 ? PAIRS : 1][SPLIT > 1 ? (SPLIT / 2) * DB * 16 * 64 : 1];  // see hand_over
  __shared__ float handed_ml[PAIRS][SPLIT > 1 ? (SPLIT / 2) * 2 * 64 : 1];
  const int q_at = wave * (QB * KS * 64) + lane;
  bf16x8* qf = q_lds + q_at;
  // the wave's two blocks start at these tokens; the later one is absent when it is the earlier one itself
  const int start[2] = {32 * w, 32 * (blocks - 1 - w)};
  const bool has_second = blocks - 1 - w > w;

  if constexpr (QB == 2) {
    int lo[2], hi[2];
    float m[2], l[2];
    f32x16 acc[2][DB];
    BlockRange range[2];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int tok = start[qb] + col;
      const bool valid = works && tok < qlen && (qb == 0 || has_second);
      const int p = p0 + tok;
      lo[qb] = valid ? (window > 0 ? max(0, p - window + 1) : 0) : 1;
      hi[qb] = valid ? p : 0;
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[(qb * KS + ks) * 64] = valid ? load8(q + (row0 + tok) * q_stride + (size_t)head * HD + 16 * ks + 8 * g) : zero8();
      m[qb] = -INFINITY;
      l[qb] = 0.f;
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[qb][b][r] = 0.f;
      range[qb] = block_range(start[qb], qlen, p0, window);
    }
    const int end = has_second ? range[1].last : range[0].last;
    src.tlo = range[0].first & ~15;
    src.thi = end & ~15;
    // the tiles of 64 keys in order: both blocks as far as the earlier one's keys reach (with a window the later
    // one may see none of them yet: they are masked), then, with a window after a gap, the later block alone
    auto after = [&](int kb) {
      int next = kb + 64;
      if (has_second && kb <= range[0].last && next > range[0].last && next + 63 < range[1].first) next = range[1].first & ~63;
      return next;
    };
    auto my_next = [&](int kb) {  // the waves of a pair (in all the workgroups that share it) take the tiles in turn
      for (int i = 0; i < SPLIT * parts; ++i) kb = after(kb);
      return kb;
    };
    int kb = range[0].first & ~63;
    for (int i = 0; i < part * SPLIT + half; ++i) kb = after(kb);
    if (!works) kb = end + 1;  // (a pair beyond the request's last block only goes to the barriers)
    load_keys<HD, T>(kf, src, kb, lane);
    load_values<HD, T>(vf, src, kb, lane);
    if (has_second) {
      while (kb <= range[0].last) {
        const int next = my_next(kb);
        const bool mask = !(range[0].unmasked(kb) && range[1].unmasked(kb));
        attend64_q32<HD, 2, 3>(m, l, acc, q_lds, q_at, kf, vf, src, kb, next, lo, hi, mask, c, lane);
        kb = next;
      }
      while (kb <= range[1].last) {
        const int next = my_next(kb);
        attend64_q32<HD, 2, 2>(m, l, acc, q_lds, q_at, kf, vf, src, kb, next, lo, hi, !range[1].unmasked(kb), c, lane);
        kb = next;
      }
    } else {
      while (kb <= range[0].last) {
        const int next = my_next(kb);
        attend64_q32<HD, 2, 1>(m, l, acc, q_lds, q_at, kf, vf, src, kb, next, lo, hi, !range[0].unmasked(kb), c, lane);
        kb = next;
      }
    }
    if constexpr (SPLIT > 1) {
#pragma unroll
      for (int qb = 0; qb < 2; ++qb)
        hand_over<DB, SPLIT>(m[qb], l[qb], acc[qb], handed[wave], handed_ml[wave], half, lane, c, qb > 0);
      if (half != 0 || !works) return;
    }
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const float total = l[qb] + __shfl_xor(l[qb], 32, kWave);
      const int tok = start[qb] + col;
      if (tok >= qlen || (qb == 1 && !has_second)) continue;
      if (parts > 1) {
        const size_t cell = ((size_t)part * n_rows + (row0 + tok - first_row)) * nh + head;
        store_part<HD>(acc[qb], m[qb], total, part_acc + cell * HD, part_ml + cell * 2, g);
        continue;
      }
      store_block<HD>(acc[qb], total, out + (row0 + tok) * out_stride + (size_t)head * HD, g);
    }
  } else {
    for (int which = 0; which < (has_second ? 2 : 1); ++which) {
      const int tok = start[which] + col;
      const bool valid = tok < qlen;
      const int p = p0 + tok;
      int lo[1] = {valid ? (window > 0 ? max(0, p - window + 1) : 0) : 1}, hi[1] = {valid ? p : 0};
      float m[1] = {-INFINITY}, l[1] = {0.f};
      f32x16 acc[1][DB];
#pragma unroll
      for (int ks = 0; ks < KS; ++ks)
        qf[ks * 64] = valid ? load8(q + (row0 + tok) * q_stride + (size_t)head * HD + 16 * ks + 8 * g) : zero8();
#pragma unroll
      for (int b = 0; b < DB; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[0][b][r] = 0.f;
      const BlockRange range = block_range(start[which], qlen, p0, window);
      src.tlo = range.first & ~15;
      src.thi = range.last & ~15;
      constexpr int SPAN = 32 * T;  // the waves of the pair take the steps of SPAN keys in turn
      const int kb0 = (range.first & ~(SPAN - 1)) + (part * SPLIT + half) * SPAN, stride = SPAN * SPLIT * parts;
      load_keys<HD, T>(kf, src, kb0, lane);
      load_values<HD, T>(vf, src, kb0, lane);
      for (int kb = kb0; kb <= range.last; kb += stride)
        attend64_q32<HD, 1, 1, T>(m, l, acc, q_lds, q_at, kf, vf, src, kb, kb + stride, lo, hi, !range.unmasked(kb, SPAN), c,
                                  lane);
      if constexpr (SPLIT > 1) {
        hand_over<DB, SPLIT>(m[0], l[0], acc[0], handed[wave], handed_ml[wave], half, lane, c, which > 0);
        if (half != 0) continue;
      }
      const float total = l[0] + __shfl_xor(l[0], 32, kWave);
      if (valid && parts > 1) {
        const size_t cell = ((size_t)part * n_rows + (row0 + tok - first_row)) * nh + head;
        store_part<HD>(acc[0], m[0], total, part_acc + cell * HD, part_ml + cell * 2, g);
      } else if (valid) {
        store_block<HD>(acc[0], total, out + (row0 + tok) * out_stride + (size_t)head * HD, g);
      }
    }
  }
}

#define GB_FOR_HEAD_SIZES(X) X(16) X(32) X(48) X(64) X(80) X(96) X(112) X(128)

}  // namespace

extern "C" int gb_attention_supported_head_size(int hd) { return hd >= 16 && hd <= 128 && hd % 16 == 0; }

// q, out: rows 0 .. n_decode-1 are the decoding requests (one row each).  ws_acc must hold
// n_decode*nh*splits*hd floats and ws_ml n_decode*nh*splits*2, with splits = ceil(max_context / chunk).
extern "C" int gb_attention_decode_bf16(const void* q, int q_stride, void* out, int out_stride, void* ws_acc, void* ws_ml,
                                        const int32_t* positions, const int32_t* tables, int table_stride,
                                        const void* k_pages, const void* v_pages, int n_decode, int nh, int nkv, int hd,
                                        int page_size, float scale, int window, int chunk, int max_context,
                                        hipStream_t stream) {
  GB_REQUIRE(n_decode >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_decode: bad head counts nh=%d nkv=%d", nh, nkv);
  GB_REQUIRE(gb_attention_supported_head_size(hd), "attention_decode: head size %d is not a multiple of 16 up to 128", hd);
  GB_REQUIRE(nh / nkv <= 16, "attention_decode: %d query heads per kv head exceed the 16 columns of a tile", nh / nkv);
  GB_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_decode: page size %d is not a multiple of 16", page_size);
  GB_REQUIRE(chunk >= 256 && chunk % 256 == 0 && max_context > 0, "attention_decode: chunk %d must be a multiple of 256", chunk);
  GB_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && out_stride % 4 == 0, "attention_decode: q rows must be 16-byte aligned");
  GB_REQUIRE(n_decode <= 65535 && nkv <= 65535, "attention_decode: too many requests or kv heads for one launch");
  if (n_decode == 0) return 0;
  const int splits = (max_context + chunk - 1) / chunk;
  // one workgroup per request and kv head (no chunks to combine afterwards) gets 16 waves, so that as
  // many loads are in flight as with four workgroups of four
  const int G = nh / nkv;
  // (not for contexts of up to 512 keys: half of the sixteen waves would find none, and four waves a workgroup put
  // more workgroups on a compute unit: 32 requests of 512 tokens, SmolLM2-1.7B shapes, 32 -> 23 us a layer)
  // (nor for heads above 64: sixteen waves of those have 128 registers each, which the larger heads do not fit
  // without spilling: Llama-3-8B shapes at 32 and 64 requests, 1,500 to 4,096 keys, 15 to 25 % faster with four)
  const int waves = (splits == 1 && max_context > 512 && hd <= 64 && 16 * (32 + (size_t)hd * G) * sizeof(float) <= 65536) ? 16 : 4;
  const size_t lds = (size_t)waves * (32 + (size_t)hd * G) * sizeof(float);
  const dim3 grid(splits, nkv, n_decode), block(waves * 64);
#define GB_CASE(HD)                                                                                                         \
  if (hd == HD) {                                                                                                           \
    if (waves == 16)                                                                                                        \
      hipLaunchKernelGGL((decode_kernel<HD, 16>), grid, block, lds, stream, (const bf16*)q, q_stride, (bf16*)out, out_stride, \
                         (float*)ws_acc, (float*)ws_ml, positions, tables, table_stride, (const bf16*)k_pages,              \
                         (const bf16*)v_pages, nh, nkv, page_size, scale, window, chunk, splits);                           \
    else                                                                                                                    \
      hipLaunchKernelGGL((decode_kernel<HD, 4>), grid, block, lds, stream, (const bf16*)q, q_stride, (bf16*)out, out_stride,  \
                         (float*)ws_acc, (float*)ws_ml, positions, tables, table_stride, (const bf16*)k_pages,              \
                         (const bf16*)v_pages, nh, nkv, page_size, scale, window, chunk, splits);                           \
  }
  GB_FOR_HEAD_SIZES(GB_CASE)
#undef GB_CASE
  if (int rc = launched("attention_decode")) return rc;
  if (splits > 1) {
    GB_REQUIRE(splits <= 256, "attention_decode: %d chunks are more than the 256 the second pass combines", splits);
    hipLaunchKernelGGL(decode_reduce_kernel, dim3(n_decode * nh), dim3(256), 0, stream, (const float*)ws_acc,
                       (const float*)ws_ml, (bf16*)out, out_stride, positions, nh, hd, window, chunk, splits);
    return launched("attention_decode_reduce");
  }
  return 0;
}

// ------------------------------------------------------- decoding without a workspace from the caller
// The chunks' partial results of gb_attention_decode_bf16 in memory that the library itself holds: a file-scope
// array on every GPU, instead of the caller's ws_acc / ws_ml.  For callers that cannot allocate.  Declared and
// described in attention_bf16.h.
namespace {
static __device__ __align__(256) float scratch[GB_DECODE_STATIC_FLOATS];
// In host code the array's name is only a handle for hipGetSymbolAddress; the address kernels may use is asked
// for once per device, with that device current, and kept here.
constexpr int kMaxDevices = 64;
float* scratch_of_device[kMaxDevices];
std::mutex scratch_lock;

int static_scratch(float** ptr) {
  int device = -1;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return fail("attention_decode_static: hipGetDevice: %s", hipGetErrorString(e));
  if (device < 0 || device >= kMaxDevices) return fail("attention_decode_static: device %d is beyond the %d this library keeps scratch for", device, kMaxDevices);
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (!scratch_of_device[device]) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) return fail("attention_decode_static: hipGetSymbolAddress on device %d: %s", device, hipGetErrorString(e));
    scratch_of_device[device] = static_cast<float*>(p);
  }
  *ptr = scratch_of_device[device];
  return 0;
}
}  // namespace

extern "C" int gb_attention_decode_bf16_static(const void* q, int q_stride, void* out, int out_stride, const int32_t* positions,
                                               const int32_t* tables, int table_stride, const void* k_pages,
                                               const void* v_pages, int n_decode, int nh, int nkv, int hd, int page_size,
                                               float scale, int window, int chunk, int max_context, hipStream_t stream) {
  GB_REQUIRE(n_decode >= 0 && nh > 0 && hd > 0 && chunk > 0 && max_context > 0, "attention_decode_static: bad sizes");
  const long long splits = ((long long)max_context + chunk - 1) / chunk;
  const long long cells = (long long)n_decode * nh * splits;
  float *ws_acc = nullptr, *ws_ml = nullptr;
  if (splits > 1) {  // one chunk a request writes its result directly: nothing is kept between the kernels
    GB_REQUIRE(cells * (hd + 2) <= (long long)GB_DECODE_STATIC_FLOATS,
               "attention_decode_static: %d requests x %d heads x %lld chunks x (%d + 2) floats = %lld exceed the %lld floats "
               "the library holds: use fewer chunks (a larger chunk), or gb_attention_decode_bf16 with a workspace",
               n_decode, nh, splits, hd, cells * (hd + 2), (long long)GB_DECODE_STATIC_FLOATS);
    float* base = nullptr;
    if (int rc = static_scratch(&base)) return rc;
    ws_acc = base;
    ws_ml = base + cells * hd;  // cells * hd floats: a multiple of 16 floats, so still 64-byte aligned
  }
  return gb_attention_decode_bf16(q, q_stride, out, out_stride, ws_acc, ws_ml, positions, tables, table_stride, k_pages, v_pages,
                                  n_decode, nh, nkv, hd, page_size, scale, window, chunk, max_context, stream);
}

// How the prompt portions of a step are spread over the chip.  A pair of blocks of 32 tokens is the unit of work.
// A compute unit is what a workgroup's waves share, and what bounds them together: so the pairs are spread over
// workgroups first (four a workgroup only if that still gives every compute unit one), then a pair's keys over
// waves (four a workgroup; eight where even single pairs leave compute units idle), and where the pairs are fewer
// than half the compute units and the contexts long, over `parts` workgroups whose sums a second pass adds.
struct PrefillPlan {
  int per_group, split, parts;
};
inline PrefillPlan prefill_plan(int max_q_len, int max_context, int nh, int n_seqs, int hd) {
  const long long pairs = (long long)((max_q_len + 63) / 64) * nh * n_seqs;
  // measured (32 heads of 64: 2,048 tokens 47.9 -> 40.7 us, 3,072 tokens 88.6 -> 79.4 with two pairs of two waves
  // each in place of four pairs; from 4,096 tokens on no gain): four pairs a workgroup once each compute unit
  // has two such workgroups
  const long long four = hd <= 64 ? 2048 : 1024;
  PrefillPlan p{pairs >= four ? 4 : pairs >= 512 ? 2 : 1, 1, 1};
  if (hd <= 64) {
    p.split = 4 / p.per_group;
    if (p.per_group == 1 && pairs <= 256) p.split = 8;  // (512 tokens of 32 heads at context 4,096: 43 -> 36 us)
  } else if (p.per_group < 4) {  // one block at a time: waves share keys only in a workgroup of one pair
    p.per_group = 1;
    p.split = pairs <= 256 ? 8 : 4;  // (512 tokens of 32 heads of 128 at context 4,096: 80 -> 67 us)
  }
  if (p.per_group == 1 && pairs <= 128) {
    // a wave keeps at least four tiles of 64 keys; four waves a workgroup then, and up to eight workgroups a pair
    const int tiles = (max(max_context, max_q_len) + 63) / 64;
    int parts = (int)(256 / (pairs > 0 ? pairs : 1));
    parts = parts > 8 ? 8 : parts;
    while (parts > 1 && parts * 4 * 4 > tiles) --parts;
    if (parts > 1) p.parts = parts, p.split = 4;
  }
  return p;
}

// Workgroups that would share a pair's keys with these sizes (1: none do); the caller then provides
// parts * rows * nh * (hd + 2) floats for their sums, rows being all rows of the portions.
extern "C" int gb_attention_prefill_parts(int max_q_len, int max_context, int nh, int n_seqs, int hd) {
  return prefill_plan(max_q_len, max_context, nh, n_seqs, hd).parts;
}

// Requests seq_base .. seq_base+n_seqs-1 of the step (prompt portions); max_q_len is the longest portion and
// max_context the longest context any of them reaches (both only shape the launch).  first_row, n_rows: the rows of
// q and out that the portions occupy (contiguous); part_ws: float32 workspace of part_floats elements, needed if
// gb_attention_prefill_parts says so.
extern "C" int gb_attention_prefill_bf16(const void* q, int q_stride, void* out, int out_stride, const int32_t* q_start,
                                         const int32_t* q_len, const int32_t* pos0, int seq_base, int n_seqs, int max_q_len,
                                         int max_context, const int32_t* tables, int table_stride, const void* k_pages,
                                         const void* v_pages, int nh, int nkv, int hd, int page_size, float scale, int window,
                                         int first_row, int n_rows, float* part_ws, long long part_floats,
                                         hipStream_t stream) {
  GB_REQUIRE(n_seqs >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_prefill: bad head counts nh=%d nkv=%d", nh, nkv);
  GB_REQUIRE(gb_attention_supported_head_size(hd), "attention_prefill: head size %d is not a multiple of 16 up to 128", hd);
  GB_REQUIRE(page_size >= 16 && (page_size & (page_size - 1)) == 0, "attention_prefill: page size %d is not a power of two from 16 up", page_size);
  int page_shift = 4;
  while ((1 << page_shift) < page_size) ++page_shift;
  GB_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && out_stride % 4 == 0 && ((uintptr_t)out % 8 == 0),
             "attention_prefill: q rows must be 16-byte aligned and out rows 8-byte aligned");
  GB_REQUIRE(n_seqs <= 65535 && nh <= 65535, "attention_prefill: too many requests or heads for one launch");
  if (n_seqs == 0 || max_q_len <= 0) return 0;
  const PrefillPlan plan = prefill_plan(max_q_len, max_context, nh, n_seqs, hd);
  const int per_group = plan.per_group, split = plan.split, parts = plan.parts;
  float *part_acc = nullptr, *part_ml = nullptr;
  if (parts > 1) {
    const long long cells = (long long)parts * n_rows * nh;
    GB_REQUIRE(part_ws && part_floats >= cells * (hd + 2) && n_rows > 0 && first_row >= 0 && ((uintptr_t)part_ws % 16 == 0),
               "attention_prefill: %d workgroups share a pair's keys: a workspace of %lld floats is needed", parts,
               cells * (hd + 2));
    part_acc = part_ws;
    part_ml = part_ws + cells * hd;
  }
  const dim3 grid((max_q_len + 64 * per_group - 1) / (64 * per_group) * parts, nh, n_seqs), block(64 * per_group * split);
#define GB_LAUNCH(HD, QB, PAIRS, SPLIT)                                                                                     \
  hipLaunchKernelGGL((prefill_kernel<HD, QB, PAIRS, SPLIT>), grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out, \
                     out_stride, q_start, q_len, pos0, seq_base, tables, table_stride, (const bf16*)k_pages,               \
                     (const bf16*)v_pages, nh, nkv, page_shift, scale, window, part_acc, part_ml, parts, first_row, n_rows)
#define GB_CASE(HD)                                        \
  if (hd == HD) {                                          \
    if constexpr (HD <= 64) {                              \
      if (split == 1) GB_LAUNCH(HD, 2, 4, 1);              \
      if (split == 2) GB_LAUNCH(HD, 2, 2, 2);              \
      if (split == 4) GB_LAUNCH(HD, 2, 1, 4);              \
      if (split == 8) GB_LAUNCH(HD, 2, 1, 8);              \
    } else {                                               \
      if (per_group == 4) GB_LAUNCH(HD, 1, 4, 1);          \
      if (per_group == 1 && split == 4) GB_LAUNCH(HD, 1, 1, 4); \
      if (per_group == 1 && split == 8) GB_LAUNCH(HD, 1, 1, 8); \
    }                                                      \
  }
  GB_FOR_HEAD_SIZES(GB_CASE)
#undef GB_CASE
#undef GB_LAUNCH
  if (int rc = launched("attention_prefill")) return rc;
  if (parts > 1) {
    hipLaunchKernelGGL(prefill_parts_kernel, dim3((unsigned)(n_rows * nh)), dim3((hd + 63) / 64 * 64), 0, stream, part_acc, part_ml,
                       (bf16*)out, out_stride, first_row, n_rows, nh, hd, parts, scale * 1.4426950408889634f);
    return launched("attention_prefill (second pass)");
  }
  return 0;
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_attention_decode_bf16)
GB_TAPED(gb_attention_prefill_bf16)
