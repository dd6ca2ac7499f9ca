// Plain paged attention, one block per (token, query head), any head size up to 256, any
// number of heads and groups, 32-bit or bfloat16 storage with 32-bit arithmetic throughout.
// It is the attention of the true 32-bit path (prompt portions and decoded tokens alike) and
// the twin that the tuned bfloat16 kernels are checked against.
//
// Token t of request s at position p reads keys lo..p of its own request through the block
// table, lo = 0 or p - window + 1 (crates/glassbox-core/src/model.rs:285-312):
//   score = dot(q, k) * scale ; prob = softmax(score) ; out = sum prob * v
//
// The order of every addition depends on the token's position alone, not on the batch and not
// on how the work is spread over workgroups.  Keys go in chunks of 256 from lo on.  A chunk is
// computed by itself: a thread a key for the scores (dot products in ascending dimension), the
// chunk's own maximum m_c, e = exp(score - m_c), their sum l_c, and sum e * v, for which a thread
// owns (dimension, word of four slots of a page) pairs and walks the chunk's pages in order, so
// that a page's values are read as whole 16-byte words by neighbouring lanes.  Chunks are then
// merged in ascending order (merge_chunk), and at the end a dimension's words are added in
// ascending order and divided by the sum.
//
// Three ways to run this, with the same bits: one workgroup walks all chunks of its (token, head)
// and merges in registers; or, for a few tokens with long contexts (a decode step, whose handful
// of workgroups would leave most of the chip idle), a workgroup a chunk writes (m_c, l_c, sums) to
// a workspace and a second kernel merges them, chunk by chunk, by the same function; or, for the
// many tokens of a prompt portion, a workgroup takes eight rows of the step: where these are one
// request's tokens at consecutive positions (and no window moves their chunks apart) they read
// the same keys and values, so a key or a word of values is loaded once and used for all eight,
// each token's own sums being what they are in the other forms; other groups of eight (where one
// request's rows end and the next one's begin) are walked one token after the other.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kChunk = 256;
constexpr int kMaxOwn = 16;   // (dimension, word) pairs a thread owns at most: head size * page size <= 16,384

struct Running {
  float m, l;
};

// (m, l, acc) of the chunks so far, joined by the next chunk's (m_c, l_c, a_c).  The same
// expressions in both kernels that merge: products and fused multiply-adds are spelled out, so
// that the compiler has no choice of how to contract them.
template <int PER>
__device__ __forceinline__ void merge_chunk(Running& r, float (&acc)[PER], float m_c, float l_c, const float (&a_c)[PER]) {
  const float m_new = fmaxf(r.m, m_c);
  const float alpha = expf(r.m - m_new);   // 0 for the first chunk (m = -inf)
  const float beta = expf(m_c - m_new);
  r.l = fmaf(l_c, beta, r.l * alpha);
#pragma unroll
  for (int u = 0; u < PER; ++u) acc[u] = fmaf(a_c[u], beta, acc[u] * alpha);
  r.m = m_new;
}

template <typename T> __device__ __forceinline__ void load_words(const T* p, float (&v)[4]);
template <> __device__ __forceinline__ void load_words<float>(const float* p, float (&v)[4]) {
  const f32x4 x = *reinterpret_cast<const f32x4*>(p);
  v[0] = x[0]; v[1] = x[1]; v[2] = x[2]; v[3] = x[3];
}
template <> __device__ __forceinline__ void load_words<bf16>(const bf16* p, float (&v)[4]) {
  const bf16x4 x = *reinterpret_cast<const bf16x4*>(p);
  v[0] = (float)x[0]; v[1] = (float)x[1]; v[2] = (float)x[2]; v[3] = (float)x[3];
}

// dot(q, key) in ascending dimension; the key lies in pieces of `piece` elements (key_offset)
template <typename T>
__device__ __forceinline__ float key_dot(const float* qs, const T* kb, int slot, int hd, int page_size, int piece) {
  float dot = 0.f;
  if (piece == 8) {
#pragma unroll 4
    for (int d0 = 0; d0 < hd; d0 += 8) {
      const T* kr = kb + ((size_t)(d0 / 8) * page_size + slot) * 8;
      float lo[4], hi[4];
      load_words<T>(kr, lo);
      load_words<T>(kr + 4, hi);
#pragma unroll
      for (int e = 0; e < 4; ++e) dot = fmaf(qs[d0 + e], lo[e], dot);
#pragma unroll
      for (int e = 0; e < 4; ++e) dot = fmaf(qs[d0 + 4 + e], hi[e], dot);
    }
  } else {
    for (int d0 = 0; d0 < hd; d0 += piece) {
      const T* kr = kb + key_offset(slot, d0, page_size, piece);
      for (int e = 0; e < piece; ++e) dot = fmaf(qs[d0 + e], to_f(kr[e]), dot);
    }
  }
  return dot;
}

struct Shape {
  int nh, nkv, hd, page_size, window, table_stride;
  float scale;
};

// One chunk by itself: keys c0 .. hi of the token's request.  Leaves m_c, l_c and the thread's sums a_c.
// `qs` holds the query, `es` (kChunk floats) and `scratch` (17) are the block's.
template <typename T, int PER>
__device__ __forceinline__ void chunk_alone(const Shape& sh, const float* qs, float* es, float* scratch,
                                            const int32_t* __restrict__ table, const T* __restrict__ k_pages,
                                            const T* __restrict__ v_pages, int kvh, int c0, int hi, float& m_c, float& l_c,
                                            float (&a_c)[PER]) {
  const int tid = threadIdx.x;
  const int ps = sh.page_size, hd = sh.hd;
  const int p = c0 + tid;
  float s = -INFINITY;
  if (p <= hi) {
    const int page = table[p / ps];
    const T* kb = k_pages + ((size_t)page * sh.nkv + kvh) * ps * hd;
    s = key_dot<T>(qs, kb, p % ps, hd, ps, key_piece(hd)) * sh.scale;
  }
  m_c = block_max(s, scratch);
  const float e = p <= hi ? expf(s - m_c) : 0.f;
  es[tid] = e;
  l_c = block_sum(e, scratch);   // also orders the writes of es before the reads below
  const int words = ps / 4, pairs = hd * words;
#pragma unroll
  for (int u = 0; u < PER; ++u) a_c[u] = 0.f;
  const int pg_last = hi / ps;
#pragma unroll 4
  for (int pg = c0 / ps; pg <= pg_last; ++pg) {
    const int page = table[pg];
    const T* vb = v_pages + ((size_t)page * sh.nkv + kvh) * hd * ps;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int idx = tid + kChunk * u;
      if (idx >= pairs) continue;
      const int d = idx / words, p0 = pg * ps + 4 * (idx % words);
      if (p0 + 3 < c0 || p0 > hi) continue;
      float v[4];
      load_words<T>(vb + (size_t)d * ps + 4 * (idx % words), v);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int pj = p0 + j;
        if (pj >= c0 && pj <= hi) a_c[u] = fmaf(es[pj - c0], v[j], a_c[u]);
      }
    }
  }
  __syncthreads();   // es is written again by the next chunk
}

// The end: a dimension's words added in ascending order, divided by the sum.
template <typename T, int PER>
__device__ __forceinline__ void finish(const Shape& sh, float* comb, const float (&acc)[PER], float l, T* out_row) {
  const int tid = threadIdx.x;
  const int words = sh.page_size / 4, pairs = sh.hd * words;
#pragma unroll
  for (int u = 0; u < PER; ++u) {
    const int idx = tid + kChunk * u;
    if (idx < pairs) comb[idx] = acc[u];
  }
  __syncthreads();
  if (tid < sh.hd) {
    float sum = 0.f;
    for (int wd = 0; wd < words; ++wd) sum += comb[tid * words + wd];
    out_row[tid] = from_f<T>(sum / l);
  }
}

__device__ __forceinline__ int ws_stride(int per) { return per * kChunk + 2; }

template <typename T, int PER, bool SPLIT>
__global__ __launch_bounds__(kChunk) void attention_plain_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tables, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, Shape sh, float* __restrict__ ws, int max_chunks) {
  extern __shared__ float smem[];
  float* qs = smem;                   // [hd]
  float* es = smem + sh.hd;           // [kChunk]
  float* scratch = es + kChunk;       // [17]
  float* comb = scratch + 17;         // [hd * page_size / 4]
  const int t = blockIdx.x / sh.nh, h = blockIdx.x % sh.nh;
  const int kvh = h / (sh.nh / sh.nkv);
  const int pos = positions[t];
  const int32_t* table = tables + (size_t)tok_seq[t] * sh.table_stride;
  const int lo = sh.window > 0 ? max(0, pos - sh.window + 1) : 0;
  const int n_chunks = (pos - lo) / kChunk + 1;
  const int tid = threadIdx.x;
  if (SPLIT && (int)blockIdx.y >= n_chunks) return;

  for (int d = tid; d < sh.hd; d += kChunk) qs[d] = to_f(q[(size_t)t * q_stride + (size_t)h * sh.hd + d]);
  __syncthreads();

  if (SPLIT) {
    const int c = blockIdx.y, c0 = lo + c * kChunk;
    float m_c, l_c, a_c[PER];
    chunk_alone<T, PER>(sh, qs, es, scratch, table, k_pages, v_pages, kvh, c0, min(c0 + kChunk - 1, pos), m_c, l_c, a_c);
    float* cell = ws + ((size_t)blockIdx.x * max_chunks + c) * ws_stride(PER);
#pragma unroll
    for (int u = 0; u < PER; ++u) cell[u * kChunk + tid] = a_c[u];
    if (tid == 0) {
      cell[PER * kChunk] = m_c;
      cell[PER * kChunk + 1] = l_c;
    }
    return;
  }
  Running r{-INFINITY, 0.f};
  float acc[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) acc[u] = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const int c0 = lo + c * kChunk;
    float m_c, l_c, a_c[PER];
    chunk_alone<T, PER>(sh, qs, es, scratch, table, k_pages, v_pages, kvh, c0, min(c0 + kChunk - 1, pos), m_c, l_c, a_c);
    merge_chunk<PER>(r, acc, m_c, l_c, a_c);
  }
  finish<T, PER>(sh, comb, acc, r.l, out + (size_t)t * out_stride + (size_t)h * sh.hd);
}

// ---- several tokens a workgroup ------------------------------------------------------------------------------
constexpr int kGroup = 8;         // rows of the step a workgroup
constexpr int kGroupMaxOwn = 4;   // (dimension, word) pairs a thread owns at most in this form

// dot(q_j, key) for Q queries, each in ascending dimension: the key's words are loaded once.  The queries are read
// where they lie in memory: their addresses are the same for every lane, so they come through the scalar unit into
// scalar registers and cost the lanes neither loads nor LDS reads.
template <typename T, int Q>
__device__ __forceinline__ void key_dots(const T* __restrict__ q0, int q_stride, const T* kb, int slot, int hd, int page_size,
                                         int piece, float (&dot)[Q]) {
#pragma unroll
  for (int j = 0; j < Q; ++j) dot[j] = 0.f;
  if (piece == 8) {
#pragma unroll 2
    for (int d0 = 0; d0 < hd; d0 += 8) {
      const T* kr = kb + ((size_t)(d0 / 8) * page_size + slot) * 8;
      float lo[4], hi[4];
      load_words<T>(kr, lo);
      load_words<T>(kr + 4, hi);
#pragma unroll
      for (int j = 0; j < Q; ++j) {
        const T* qj = q0 + (size_t)j * q_stride + d0;
#pragma unroll
        for (int e = 0; e < 4; ++e) dot[j] = fmaf(to_f(qj[e]), lo[e], dot[j]);
#pragma unroll
        for (int e = 0; e < 4; ++e) dot[j] = fmaf(to_f(qj[4 + e]), hi[e], dot[j]);
      }
    }
  } else {
    for (int d0 = 0; d0 < hd; d0 += piece) {
      const T* kr = kb + key_offset(slot, d0, page_size, piece);
      for (int e = 0; e < piece; ++e) {
        const float kv = to_f(kr[e]);
#pragma unroll
        for (int j = 0; j < Q; ++j) dot[j] = fmaf(to_f(q0[(size_t)j * q_stride + d0 + e]), kv, dot[j]);
      }
    }
  }
}

// block_max and block_sum (common.h) of Q values at once: the same sums in the same order, every
// thread adding the waves' parts for itself.  `scratch` holds Q * 4 floats.
template <int Q, bool MAX>
__device__ __forceinline__ void block_reduce(float (&v)[Q], float* scratch) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int j = 0; j < Q; ++j) v[j] = MAX ? wave_max(v[j]) : wave_sum(v[j]);
  __syncthreads();
  if (lane == 0) {
#pragma unroll
    for (int j = 0; j < Q; ++j) scratch[j * 4 + wave] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    if (MAX) {
      float t = scratch[j * 4];
      for (int w = 1; w < kChunk / kWave; ++w) t = fmaxf(t, scratch[j * 4 + w]);
      v[j] = t;
    } else {
      float t = 0.f;
      for (int w = 0; w < kChunk / kWave; ++w) t += scratch[j * 4 + w];
      v[j] = t;
    }
  }
}
static_assert(kChunk / kWave == 4, "block_reduce keeps four waves' parts a value");

// chunk_alone for Q tokens of one request that read the same pages: token j reads keys c0 .. hi[j], hi ascending.
// A token whose hi lies below c0 has no key here: its m_c is -inf and its sums are zero, and the caller skips it.
template <typename T, int PER, int Q>
__device__ __forceinline__ void chunk_together(const Shape& sh, const T* __restrict__ q0, int q_stride, float* es, float* scratch,
                                               const int32_t* __restrict__ table, const T* __restrict__ k_pages,
                                               const T* __restrict__ v_pages, int kvh, int c0, const int (&hi)[Q],
                                               float (&m_c)[Q], float (&l_c)[Q], float (&a_c)[Q][PER]) {
  const int tid = threadIdx.x;
  const int ps = sh.page_size, hd = sh.hd;
  const int p = c0 + tid;
  const int top = hi[Q - 1];
  float s[Q];
#pragma unroll
  for (int j = 0; j < Q; ++j) s[j] = -INFINITY;
  if (p <= top) {
    const int page = table[p / ps];
    const T* kb = k_pages + ((size_t)page * sh.nkv + kvh) * ps * hd;
    float dot[Q];
    key_dots<T, Q>(q0, q_stride, kb, p % ps, hd, ps, key_piece(hd), dot);
#pragma unroll
    for (int j = 0; j < Q; ++j)
      if (p <= hi[j]) s[j] = dot[j] * sh.scale;
  }
#pragma unroll
  for (int j = 0; j < Q; ++j) m_c[j] = s[j];
  block_reduce<Q, true>(m_c, scratch);
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    const float e = p <= hi[j] ? expf(s[j] - m_c[j]) : 0.f;
    es[j * kChunk + tid] = e;
    l_c[j] = e;
  }
  block_reduce<Q, false>(l_c, scratch);   // also orders the writes of es before the reads below
  const int words = ps / 4, pairs = hd * words;
#pragma unroll
  for (int j = 0; j < Q; ++j)
#pragma unroll
    for (int u = 0; u < PER; ++u) a_c[j][u] = 0.f;
  const int pg_last = top / ps;
#pragma unroll 4
  for (int pg = c0 / ps; pg <= pg_last; ++pg) {
    const int page = table[pg];
    const T* vb = v_pages + ((size_t)page * sh.nkv + kvh) * hd * ps;
#pragma unroll
    for (int u = 0; u < PER; ++u) {
      const int idx = tid + kChunk * u;
      if (idx >= pairs) continue;
      const int d = idx / words, p0 = pg * ps + 4 * (idx % words);
      if (p0 + 3 < c0 || p0 > top) continue;
      float v[4];
      load_words<T>(vb + (size_t)d * ps + 4 * (idx % words), v);
#pragma unroll
      for (int j = 0; j < Q; ++j) {
        // c0 and p0 are multiples of four here: the word's four weights are one 16-byte word of es
        const f32x4 e4 = *reinterpret_cast<const f32x4*>(&es[j * kChunk + p0 - c0]);
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (p0 + i <= hi[j]) a_c[j][u] = fmaf(e4[i], v[i], a_c[j][u]);
      }
    }
  }
  __syncthreads();   // es is written again by the next chunk
}

// Rows first .. first + Q - 1 of the step, one request's tokens at positions pos0 .. pos0 + Q - 1, no window.
template <typename T, int PER, int Q>
__device__ __forceinline__ void walk_together(const Shape& sh, const T* __restrict__ q0, int q_stride, float* es, float* scratch,
                                              float* comb,
                                              const int32_t* __restrict__ table, const T* __restrict__ k_pages,
                                              const T* __restrict__ v_pages, int kvh, int h, int pos0, T* __restrict__ out,
                                              int out_stride, int first) {
  Running r[Q];
  float acc[Q][PER];
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    r[j] = Running{-INFINITY, 0.f};
#pragma unroll
    for (int u = 0; u < PER; ++u) acc[j][u] = 0.f;
  }
  const int n_chunks = (pos0 + Q - 1) / kChunk + 1;
  for (int c = 0; c < n_chunks; ++c) {
    const int c0 = c * kChunk;
    int hi[Q];
#pragma unroll
    for (int j = 0; j < Q; ++j) hi[j] = min(c0 + kChunk - 1, pos0 + j);
    float m_c[Q], l_c[Q], a_c[Q][PER];
    chunk_together<T, PER, Q>(sh, q0, q_stride, es, scratch, table, k_pages, v_pages, kvh, c0, hi, m_c, l_c, a_c);
#pragma unroll
    for (int j = 0; j < Q; ++j)
      if (c0 <= pos0 + j) merge_chunk<PER>(r[j], acc[j], m_c[j], l_c[j], a_c[j]);
  }
#pragma unroll
  for (int j = 0; j < Q; ++j) {
    finish<T, PER>(sh, comb, acc[j], r[j].l, out + (size_t)(first + j) * out_stride + (size_t)h * sh.hd);
    __syncthreads();   // comb is written again for the next token
  }
}

template <typename T, int PER>
__global__ __launch_bounds__(kChunk) void attention_plain_group_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tables, const T* __restrict__ k_pages,
    const T* __restrict__ v_pages, Shape sh, int n) {
  extern __shared__ float smem[];
  float* qs = smem;                          // [kGroup][hd]
  float* es = qs + kGroup * sh.hd;           // [kGroup][kChunk]
  float* scratch = es + kGroup * kChunk;     // [kGroup * 4], and 17 for the one-token form
  float* comb = scratch + kGroup * 4 + 17;   // [hd * page_size / 4]
  const int g = blockIdx.x / sh.nh, h = blockIdx.x % sh.nh;
  const int kvh = h / (sh.nh / sh.nkv);
  const int first = g * kGroup, count = min(kGroup, n - first);
  const int tid = threadIdx.x;
  const int pos0 = positions[first], seq0 = tok_seq[first];
  bool together = count == kGroup && sh.window == 0;
  for (int j = 1; j < count; ++j) together = together && tok_seq[first + j] == seq0 && positions[first + j] == pos0 + j;

  if (together) {
    walk_together<T, PER, kGroup>(sh, q + (size_t)first * q_stride + (size_t)h * sh.hd, q_stride, es, scratch, comb,
                                  tables + (size_t)seq0 * sh.table_stride, k_pages, v_pages, kvh, h, pos0, out, out_stride, first);
    return;
  }
  for (int e = tid; e < count * sh.hd; e += kChunk) {
    const int j = e / sh.hd, d = e % sh.hd;
    qs[e] = to_f(q[(size_t)(first + j) * q_stride + (size_t)h * sh.hd + d]);
  }
  __syncthreads();
  for (int j = 0; j < count; ++j) {   // one after the other, as a workgroup of the one-token form would
    const int t = first + j;
    const int pos = positions[t];
    const int32_t* table = tables + (size_t)tok_seq[t] * sh.table_stride;
    const int lo = sh.window > 0 ? max(0, pos - sh.window + 1) : 0;
    const int n_chunks = (pos - lo) / kChunk + 1;
    Running r{-INFINITY, 0.f};
    float acc[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) acc[u] = 0.f;
    for (int c = 0; c < n_chunks; ++c) {
      const int c0 = lo + c * kChunk;
      float m_c, l_c, a_c[PER];
      chunk_alone<T, PER>(sh, qs + j * sh.hd, es, scratch + kGroup * 4, table, k_pages, v_pages, kvh, c0,
                          min(c0 + kChunk - 1, pos), m_c, l_c, a_c);
      merge_chunk<PER>(r, acc, m_c, l_c, a_c);
    }
    finish<T, PER>(sh, comb, acc, r.l, out + (size_t)t * out_stride + (size_t)h * sh.hd);
    __syncthreads();   // comb is written again for the next token
  }
}

// Merges what the workgroups of a (token, head) left, chunk by chunk in ascending order.
template <typename T, int PER>
__global__ __launch_bounds__(kChunk) void attention_plain_merge_kernel(T* __restrict__ out, int out_stride,
                                                                       const int32_t* __restrict__ positions, Shape sh,
                                                                       const float* __restrict__ ws, int max_chunks) {
  extern __shared__ float smem[];   // [hd * page_size / 4]
  const int t = blockIdx.x / sh.nh, h = blockIdx.x % sh.nh;
  const int pos = positions[t];
  const int lo = sh.window > 0 ? max(0, pos - sh.window + 1) : 0;
  const int n_chunks = min((pos - lo) / kChunk + 1, max_chunks);   // (never beyond what the workspace holds)
  const int tid = threadIdx.x;
  Running r{-INFINITY, 0.f};
  float acc[PER];
#pragma unroll
  for (int u = 0; u < PER; ++u) acc[u] = 0.f;
  for (int c = 0; c < n_chunks; ++c) {
    const float* cell = ws + ((size_t)blockIdx.x * max_chunks + c) * ws_stride(PER);
    float a_c[PER];
#pragma unroll
    for (int u = 0; u < PER; ++u) a_c[u] = cell[u * kChunk + tid];
    merge_chunk<PER>(r, acc, cell[PER * kChunk], cell[PER * kChunk + 1], a_c);
  }
  finish<T, PER>(sh, smem, acc, r.l, out + (size_t)t * out_stride + (size_t)h * sh.hd);
}

inline int own_pairs(int hd, int page_size) {
  const int per = (hd * (page_size / 4) + kChunk - 1) / kChunk;
  for (int p = 1; p <= kMaxOwn; p *= 2)
    if (per <= p) return p;
  return 0;
}

template <typename T, int PER>
void launch(const void* q, int q_stride, void* out, int out_stride, const int32_t* positions, const int32_t* tok_seq,
            const int32_t* tables, const void* k_pages, const void* v_pages, int n, const Shape& sh, float* ws,
            int max_chunks, bool grouped_form, hipStream_t stream) {
  const size_t comb = sizeof(float) * sh.hd * (sh.page_size / 4);
  const size_t smem = sizeof(float) * (sh.hd + kChunk + 17) + comb;
  if (ws != nullptr) {
    hipLaunchKernelGGL((attention_plain_kernel<T, PER, true>), dim3((unsigned)(n * sh.nh), (unsigned)max_chunks), dim3(kChunk),
                       smem, stream, (const T*)q, q_stride, (T*)out, out_stride, positions, tok_seq, tables,
                       (const T*)k_pages, (const T*)v_pages, sh, ws, max_chunks);
    hipLaunchKernelGGL((attention_plain_merge_kernel<T, PER>), dim3((unsigned)(n * sh.nh)), dim3(kChunk), comb, stream,
                       (T*)out, out_stride, positions, sh, (const float*)ws, max_chunks);
  } else if (grouped_form && PER <= kGroupMaxOwn && sh.window == 0) {   // (elsewhere the one-token form: the same bits)
    if constexpr (PER <= kGroupMaxOwn) {
      const size_t grouped = sizeof(float) * (kGroup * (sh.hd + kChunk + 4) + 17) + comb;
      const int groups = (n + kGroup - 1) / kGroup;
      hipLaunchKernelGGL((attention_plain_group_kernel<T, PER>), dim3((unsigned)(groups * sh.nh)), dim3(kChunk), grouped, stream,
                         (const T*)q, q_stride, (T*)out, out_stride, positions, tok_seq, tables, (const T*)k_pages,
                         (const T*)v_pages, sh, n);
    }
  } else {
    hipLaunchKernelGGL((attention_plain_kernel<T, PER, false>), dim3((unsigned)(n * sh.nh)), dim3(kChunk), smem, stream,
                       (const T*)q, q_stride, (T*)out, out_stride, positions, tok_seq, tables, (const T*)k_pages,
                       (const T*)v_pages, sh, nullptr, 0);
  }
}

template <typename T>
int launch_by_pairs(int per, const void* q, int q_stride, void* out, int out_stride, const int32_t* positions,
                    const int32_t* tok_seq, const int32_t* tables, const void* k_pages, const void* v_pages, int n,
                    const Shape& sh, float* ws, int max_chunks, bool grouped_form, hipStream_t stream) {
#define GB_PLAIN_CASE(P)                                                                                              \
  case P:                                                                                                             \
    launch<T, P>(q, q_stride, out, out_stride, positions, tok_seq, tables, k_pages, v_pages, n, sh, ws, max_chunks,       \
                 grouped_form, stream);                                                                               \
    break;
  switch (per) {
    GB_PLAIN_CASE(1) GB_PLAIN_CASE(2) GB_PLAIN_CASE(4) GB_PLAIN_CASE(8) GB_PLAIN_CASE(16)
    default: return fail("attention_plain: no kernel for %d pairs a thread", per);
  }
#undef GB_PLAIN_CASE
  return launched("attention_plain");
}

}  // namespace

// Floats of workspace that the chunk-by-chunk form needs for n tokens whose longest context (keys a token reads) is
// max_context, or 0 where the sizes are refused anyway.
extern "C" long long gb_attention_plain_split_floats(int n, int nh, int hd, int page_size, int max_context) {
  if (n <= 0 || nh <= 0 || hd <= 0 || page_size <= 0 || page_size % 4 || max_context <= 0) return 0;
  const int per = own_pairs(hd, page_size);
  if (per == 0) return 0;
  const long long chunks = (max_context + kChunk - 1) / kChunk;
  return (long long)n * nh * chunks * (per * kChunk + 2);
}

// ws = nullptr: a workgroup a (token, head) walks the whole context.  Otherwise ws holds at least
// gb_attention_plain_split_floats(n, nh, hd, page_size, max_context) floats, max_context is at least the most keys any
// of the tokens reads, and a workgroup a chunk of 256 keys leaves its part there for a second kernel to merge: the
// same bits, for steps of few tokens with long contexts.  grouped != 0 (without ws): eight rows a workgroup, for rows
// that are mostly portions of prompts (consecutive tokens of a request): the same bits again.
extern "C" int gb_attention_plain(const void* q, int q_stride, void* out, int out_stride, int dtype,
                                  const int32_t* positions, const int32_t* tok_seq, const int32_t* tables,
                                  int table_stride, const void* k_pages, const void* v_pages, int n, int nh, int nkv,
                                  int hd, int page_size, float scale, int window, float* ws, long long ws_floats,
                                  int max_context, int grouped, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_plain: bad sizes n=%d nh=%d nkv=%d hd=%d", n, nh, nkv, hd);
  GB_REQUIRE(nh % nkv == 0, "attention_plain: %d query heads are not a multiple of %d key heads", nh, nkv);
  GB_REQUIRE(hd <= kChunk, "attention_plain: head size %d is above the supported 256", hd);
  GB_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd, "attention_plain: row strides shorter than the heads");
  GB_REQUIRE(page_size > 0 && table_stride > 0 && window >= 0, "attention_plain: bad page size, table stride or window");
  GB_REQUIRE(page_size % 4 == 0, "attention_plain: a page of %d tokens is not whole words of four slots", page_size);
  GB_REQUIRE((long long)n * nh < (1ll << 31), "attention_plain: too many (token, head) pairs");
  const int per = own_pairs(hd, page_size);
  GB_REQUIRE(per != 0, "attention_plain: head size %d times page size %d is above %d", hd, page_size, kMaxOwn * kChunk * 4);
  GB_REQUIRE(!(grouped && ws != nullptr), "attention_plain: several rows a workgroup and a workgroup a chunk exclude each other");
  if (n == 0) return 0;
  int max_chunks = 0;
  if (ws != nullptr) {
    GB_REQUIRE(max_context > 0, "attention_plain: the chunk-by-chunk form needs the longest context");
    max_chunks = (max_context + kChunk - 1) / kChunk;
    GB_REQUIRE(max_chunks <= 65535, "attention_plain: a context of %d keys is more chunks than a launch takes", max_context);
    GB_REQUIRE(ws_floats >= gb_attention_plain_split_floats(n, nh, hd, page_size, max_context),
               "attention_plain: the workspace holds %lld floats, %lld are needed", ws_floats,
               gb_attention_plain_split_floats(n, nh, hd, page_size, max_context));
  }
  const Shape sh{nh, nkv, hd, page_size, window, table_stride, scale};
  if (dtype == kF32)
    return launch_by_pairs<float>(per, q, q_stride, out, out_stride, positions, tok_seq, tables, k_pages, v_pages, n, sh, ws,
                                  max_chunks, grouped != 0, stream);
  if (dtype == kBF16)
    return launch_by_pairs<bf16>(per, q, q_stride, out, out_stride, positions, tok_seq, tables, k_pages, v_pages, n, sh, ws,
                                 max_chunks, grouped != 0, stream);
  return fail("attention_plain: unknown dtype %d", dtype);
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_attention_plain)
