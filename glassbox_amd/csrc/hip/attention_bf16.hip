// Paged attention in bfloat16 on the matrix cores, for decoding and for prompt portions.
//
// Per request and kv head the work is out[col] = softmax(q[col] . K^T * scale) . V for up to 16
// "columns" that share the keys: when decoding, the columns are the query heads of one token that
// map to the kv head (grouped-query attention reads each key once for the whole group); for a
// prompt portion they are 16 consecutive tokens of one query head.  Both use the same inner step
// over 64 keys:
//   S^T[key, col] = K[key, :] . Q[col, :]     v_mfma_f32_16x16x32_bf16, A = 16 keys x 32 dims straight
//                                             from the key page (16 bytes a lane), B = the query columns
//   running max / sum per column in 32-bit, keys outside [lo, hi] of the column masked to -inf
//   O^T[dim, col] += V^T[dim, key] . P^T[key, col]   A = 16 dims x 32 keys from the transposed value
//                                             page (8 bytes a lane from each of two tiles), B = the
//                                             probabilities, taken from the score registers as they
//                                             are (the k order of both operands is permuted alike)
// so neither scores nor probabilities pass through LDS, and keys and values go from memory into
// MFMA operands directly.  Pages: keys [page][kv head][slot][hd], values [page][kv head][hd][slot].
//
// Decoding splits a request's context into chunks of a multiple of 256 keys, one workgroup per
// (chunk, kv head, request), four waves taking 64 keys each in turn; partial results are merged
// in a fixed order (waves in LDS, chunks by a second kernel), so the result is the same on every
// run.  crates/glassbox-core/src/model.rs:285-312 is the formula.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x4 load4(const bf16* p) { return *reinterpret_cast<const bf16x4*>(p); }
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
    const bf16* kb = kp + (((size_t)page * nkv + kvh) * P + slot0 + j) * HD;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int d0 = ks * 32 + c * 8;
      kf[t][ks] = d0 < HD ? load8(kb + d0) : zero8();
    }
    const bf16* vb = vp + ((size_t)page * nkv + kvh) * HD * P + slot0 + 4 * c;
#pragma unroll
    for (int b = 0; b < DB; ++b) vf[b][t] = load4(vb + (size_t)(16 * b + j) * P);
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
template <int HD>
__global__ __launch_bounds__(256) void decode_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                                     int out_stride, float* __restrict__ ws_acc, float* __restrict__ ws_ml,
                                                     const int32_t* __restrict__ positions, const int32_t* __restrict__ tables,
                                                     int table_stride, const bf16* __restrict__ kp, const bf16* __restrict__ vp,
                                                     int nh, int nkv, int P, float scale, int window, int chunk, int splits) {
  constexpr int KS = (HD + 31) / 32, DB = HD / 16;
  __shared__ float sm_m[4][16], sm_l[4][16];
  __shared__ float sm_acc[4][HD][16];
  const int s = blockIdx.z, kvh = blockIdx.y, split = blockIdx.x;
  const int G = nh / nkv;
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
  for (int kb = c0 + wave * 64; kb < end; kb += 256) {
    if (kb + 64 <= lo) continue;
    attend64<HD>(st, qf, kp, vp, table, nkv, kvh, P, kb, col_lo, col_hi, lo, pos, scale, lane);
  }
  st.l += __shfl_xor(st.l, 16, kWave);
  st.l += __shfl_xor(st.l, 32, kWave);
  if (lane < 16) {
    sm_m[wave][col] = st.m;
    sm_l[wave][col] = st.l;
  }
#pragma unroll
  for (int b = 0; b < DB; ++b)
#pragma unroll
    for (int r = 0; r < 4; ++r) sm_acc[wave][16 * b + 4 * (lane >> 4) + r][col] = st.acc[b][r];
  __syncthreads();
  // the four waves' partial results, combined in wave order
  for (int cell = tid; cell < HD * 16; cell += 256) {
    const int d = cell >> 4, cc = cell & 15;
    if (cc >= G) continue;
    float M = sm_m[0][cc];
#pragma unroll
    for (int w = 1; w < 4; ++w) M = fmaxf(M, sm_m[w][cc]);
    float val = 0.f, L = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float f = sm_m[w][cc] == -INFINITY ? 0.f : __expf(sm_m[w][cc] - M);
      val += sm_acc[w][d][cc] * f;
      L += sm_l[w][cc] * f;
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

// One block per (request, head): the chunks' partial results, combined in chunk order.
__global__ void decode_reduce_kernel(const float* __restrict__ ws_acc, const float* __restrict__ ws_ml,
                                     bf16* __restrict__ out, int out_stride, const int32_t* __restrict__ positions, int nh,
                                     int hd, int window, int chunk, int splits) {
  const int s = blockIdx.x / nh, head = blockIdx.x % nh;
  const int pos = positions[s];
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int first = lo / chunk, last = pos / chunk;
  const size_t base = ((size_t)s * nh + head) * splits;
  float M = -INFINITY;
  for (int k = first; k <= last; ++k) M = fmaxf(M, ws_ml[(base + k) * 2]);
  for (int d = threadIdx.x; d < hd; d += blockDim.x) {
    float val = 0.f, L = 0.f;
    for (int k = first; k <= last; ++k) {
      const float f = __expf(ws_ml[(base + k) * 2] - M);
      val += ws_acc[(base + k) * hd + d] * f;
      L += ws_ml[(base + k) * 2 + 1] * f;
    }
    out[(size_t)s * out_stride + (size_t)head * hd + d] = (bf16)(val / L);
  }
}

// ---------------------------------------------------------------------------- prefill
// grid (tiles of 64 tokens, query heads, requests from seq_base on); a wave takes 16 tokens.
template <int HD>
__global__ __launch_bounds__(256) void prefill_kernel(const bf16* __restrict__ q, int q_stride, bf16* __restrict__ out,
                                                      int out_stride, const int32_t* __restrict__ q_start,
                                                      const int32_t* __restrict__ q_len, const int32_t* __restrict__ pos0,
                                                      int seq_base, const int32_t* __restrict__ tables, int table_stride,
                                                      const bf16* __restrict__ kp, const bf16* __restrict__ vp, int nh, int nkv,
                                                      int P, float scale, int window) {
  constexpr int KS = (HD + 31) / 32, DB = HD / 16;
  const int seq = seq_base + blockIdx.z, head = blockIdx.y;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int qlen = q_len[seq];
  const int t0 = blockIdx.x * 64 + wave * 16;
  if (t0 >= qlen) return;
  const int col = lane & 15, c = lane >> 4;
  const int tok = t0 + col;
  const bool valid = tok < qlen;
  const int p0 = pos0[seq];
  const int p = p0 + tok;
  const size_t row = (size_t)q_start[seq] + tok;
  const int kvh = head / (nh / nkv);
  const int32_t* table = tables + (size_t)seq * table_stride;

  bf16x8 qf[KS];
#pragma unroll
  for (int ks = 0; ks < KS; ++ks) {
    const int d0 = ks * 32 + c * 8;
    qf[ks] = (valid && d0 < HD) ? load8(q + row * q_stride + (size_t)head * HD + d0) : zero8();
  }
  Running<HD> st;
  reset(st);
  const int col_lo = valid ? (window > 0 ? max(0, p - window + 1) : 0) : 1, col_hi = valid ? p : 0;
  const int wave_hi = p0 + min(t0 + 15, qlen - 1);
  const int wave_lo = window > 0 ? max(0, p0 + t0 - window + 1) : 0;
  for (int kb = wave_lo & ~63; kb <= wave_hi; kb += 64)
    attend64<HD>(st, qf, kp, vp, table, nkv, kvh, P, kb, col_lo, col_hi, wave_lo, wave_hi, scale, lane);
  st.l += __shfl_xor(st.l, 16, kWave);
  st.l += __shfl_xor(st.l, 32, kWave);
  if (!valid) return;
  const float inv = 1.0f / st.l;
  bf16* orow = out + row * out_stride + (size_t)head * HD;
#pragma unroll
  for (int b = 0; b < DB; ++b) {
    bf16x4 o;
#pragma unroll
    for (int r = 0; r < 4; ++r) o[r] = (bf16)(st.acc[b][r] * inv);
    *reinterpret_cast<bf16x4*>(orow + 16 * b + 4 * c) = o;
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
  const dim3 grid(splits, nkv, n_decode), block(256);
#define GB_CASE(HD)                                                                                                        \
  if (hd == HD)                                                                                                            \
    hipLaunchKernelGGL(decode_kernel<HD>, grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out, out_stride,         \
                       (float*)ws_acc, (float*)ws_ml, positions, tables, table_stride, (const bf16*)k_pages,               \
                       (const bf16*)v_pages, nh, nkv, page_size, scale, window, chunk, splits);
  GB_FOR_HEAD_SIZES(GB_CASE)
#undef GB_CASE
  if (int rc = launched("attention_decode")) return rc;
  if (splits > 1) {
    hipLaunchKernelGGL(decode_reduce_kernel, dim3(n_decode * nh), dim3(64), 0, stream, (const float*)ws_acc,
                       (const float*)ws_ml, (bf16*)out, out_stride, positions, nh, hd, window, chunk, splits);
    return launched("attention_decode_reduce");
  }
  return 0;
}

// Requests seq_base .. seq_base+n_seqs-1 of the step (prompt portions); max_q_len is the longest portion.
extern "C" int gb_attention_prefill_bf16(const void* q, int q_stride, void* out, int out_stride, const int32_t* q_start,
                                         const int32_t* q_len, const int32_t* pos0, int seq_base, int n_seqs, int max_q_len,
                                         const int32_t* tables, int table_stride, const void* k_pages, const void* v_pages,
                                         int nh, int nkv, int hd, int page_size, float scale, int window, hipStream_t stream) {
  GB_REQUIRE(n_seqs >= 0 && nh > 0 && nkv > 0 && nh % nkv == 0, "attention_prefill: bad head counts nh=%d nkv=%d", nh, nkv);
  GB_REQUIRE(gb_attention_supported_head_size(hd), "attention_prefill: head size %d is not a multiple of 16 up to 128", hd);
  GB_REQUIRE(page_size >= 16 && page_size % 16 == 0, "attention_prefill: page size %d is not a multiple of 16", page_size);
  GB_REQUIRE(q_stride % 8 == 0 && ((uintptr_t)q % 16 == 0) && out_stride % 4 == 0 && ((uintptr_t)out % 8 == 0),
             "attention_prefill: q rows must be 16-byte aligned and out rows 8-byte aligned");
  GB_REQUIRE(n_seqs <= 65535 && nh <= 65535, "attention_prefill: too many requests or heads for one launch");
  if (n_seqs == 0 || max_q_len <= 0) return 0;
  const dim3 grid((max_q_len + 63) / 64, nh, n_seqs), block(256);
#define GB_CASE(HD)                                                                                                        \
  if (hd == HD)                                                                                                            \
    hipLaunchKernelGGL(prefill_kernel<HD>, grid, block, 0, stream, (const bf16*)q, q_stride, (bf16*)out, out_stride,        \
                       q_start, q_len, pos0, seq_base, tables, table_stride, (const bf16*)k_pages, (const bf16*)v_pages, nh, \
                       nkv, page_size, scale, window);
  GB_FOR_HEAD_SIZES(GB_CASE)
#undef GB_CASE
  return launched("attention_prefill");
}
