// Memory-bound parts of a decoder step, in 32-bit and bfloat16 storage: embedding
// gather, RMS norm, rotary table, rotation fused with the cache write, SiLU-multiply,
// and page copies.  All arithmetic is 32-bit; only loads and stores differ by type.
#include <type_traits>

#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

// ---------------------------------------------------------------- embedding gather
// x[i, :] = table[ids[i], :]   (crates/glassbox-core/src/model.rs:228-231)
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int32_t* __restrict__ ids, float* __restrict__ x,
                             int d, int vocab) {
  const int i = blockIdx.x;
  int id = ids[i];
  const bool ok = id >= 0 && id < vocab;
  const T* row = table + (size_t)(ok ? id : 0) * d;
  for (int c = threadIdx.x; c < d; c += blockDim.x)
    x[(size_t)i * d + c] = ok ? to_f(row[c]) : __builtin_nanf("");  // a bad id must not pass silently
}

extern "C" int gb_embed(const void* table, int table_dtype, const int32_t* ids, float* x, int n, int d, int vocab,
                        hipStream_t stream) {
  GB_REQUIRE(n >= 0 && d > 0 && vocab > 0, "embed: bad sizes n=%d d=%d vocab=%d", n, d, vocab);
  if (n == 0) return 0;
  const int threads = d >= 256 ? 256 : 64;
  if (table_dtype == kF32)
    hipLaunchKernelGGL(embed_kernel<float>, dim3(n), dim3(threads), 0, stream, (const float*)table, ids, x, d, vocab);
  else if (table_dtype == kBF16)
    hipLaunchKernelGGL(embed_kernel<bf16>, dim3(n), dim3(threads), 0, stream, (const bf16*)table, ids, x, d, vocab);
  else
    return fail("embed: unknown table dtype %d", table_dtype);
  return launched("embed");
}

// ------------------------------------------------------------------------ RMS norm
// ms = sum(x^2)/d ; s = 1/sqrt(ms + eps) ; out = g * (x * s)     (model.rs:94-100)
// One block per output row; `rows` (optional) picks the input row of each output row.
// A thread keeps its VPT values of the row (and of gamma) in registers across the reduction, so the
// row is read once and the loads of gamma overlap the sum; rows longer than VPT * threads are read
// a second time.  The sum's order is fixed by the thread layout.
template <typename G, typename O, int VPT>
__global__ void rmsnorm_kernel(const float* __restrict__ x, const G* __restrict__ gamma, const int32_t* __restrict__ rows,
                               O* __restrict__ out, int d, float eps) {
  __shared__ float partial[16];
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * d;
  float v[VPT], g[VPT];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = tid + j * nt;
    v[j] = c < d ? xr[c] : 0.f;
    g[j] = c < d ? to_f(gamma[c]) : 0.f;
  }
#pragma unroll
  for (int j = 0; j < VPT; ++j) ss += v[j] * v[j];
  for (int c = tid + VPT * nt; c < d; c += nt) {
    const float t = xr[c];
    ss += t * t;
  }
  ss = wave_sum(ss);
  if (tid % kWave == 0) partial[tid / kWave] = ss;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < (nt + kWave - 1) / kWave; ++w) total += partial[w];
  const float s = 1.0f / sqrtf(total / (float)d + eps);
  O* orow = out + (size_t)r * d;
#pragma unroll
  for (int j = 0; j < VPT; ++j) {
    const int c = tid + j * nt;
    if (c < d) orow[c] = from_f<O>(g[j] * (v[j] * s));
  }
  for (int c = tid + VPT * nt; c < d; c += nt) orow[c] = from_f<O>(to_f(gamma[c]) * (xr[c] * s));
}

// The same with four neighbouring columns a thread as one word (rows of a multiple of 4 columns, up to
// 4 * V4 * threads of them): a quarter of the loads and stores.
template <typename G, typename O, int V4>
__global__ void rmsnorm_words_kernel(const float* __restrict__ x, const G* __restrict__ gamma, const int32_t* __restrict__ rows,
                                     O* __restrict__ out, int d, float eps) {
  __shared__ float partial[16];
  const int r = blockIdx.x, tid = threadIdx.x, nt = blockDim.x;
  const float* xr = x + (size_t)(rows ? rows[r] : r) * d;
  f32x4 v[V4], g[V4];
  float ss = 0.f;
#pragma unroll
  for (int j = 0; j < V4; ++j) {
    const int c = (tid + j * nt) * 4;
    v[j] = f32x4{0.f, 0.f, 0.f, 0.f};
    g[j] = v[j];
    if (c < d) {
      v[j] = *reinterpret_cast<const f32x4*>(xr + c);
      if constexpr (std::is_same<G, float>::value) {
        g[j] = *reinterpret_cast<const f32x4*>(gamma + c);
      } else {
        const bf16x4 gb = *reinterpret_cast<const bf16x4*>(gamma + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) g[j][e] = (float)gb[e];
      }
    }
  }
#pragma unroll
  for (int j = 0; j < V4; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) ss += v[j][e] * v[j][e];
  ss = wave_sum(ss);
  if (tid % kWave == 0) partial[tid / kWave] = ss;
  __syncthreads();
  float total = 0.f;
  for (int w = 0; w < (nt + kWave - 1) / kWave; ++w) total += partial[w];
  const float s = 1.0f / sqrtf(total / (float)d + eps);
  O* orow = out + (size_t)r * d;
#pragma unroll
  for (int j = 0; j < V4; ++j) {
    const int c = (tid + j * nt) * 4;
    if (c >= d) continue;
    if constexpr (std::is_same<O, float>::value) {
      f32x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = g[j][e] * (v[j][e] * s);
      *reinterpret_cast<f32x4*>(orow + c) = o;
    } else {
      bf16x4 o;
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = (bf16)(g[j][e] * (v[j][e] * s));
      *reinterpret_cast<bf16x4*>(orow + c) = o;
    }
  }
}

extern "C" int gb_rmsnorm(const float* x, const void* gamma, int gamma_dtype, const int32_t* rows, void* out,
                          int out_dtype, int m, int d, float eps, hipStream_t stream) {
  GB_REQUIRE(m >= 0 && d > 0, "rmsnorm: bad sizes m=%d d=%d", m, d);
  if (m == 0) return 0;
  const int threads = d >= 1024 ? 256 : (d >= 256 ? 128 : 64);
  const int per_thread = (d + threads - 1) / threads;
  // whole words where the rows allow it (every row then starts at a multiple of 16 bytes)
  const bool words = d % 4 == 0 && d <= 4 * 8 * threads && (uintptr_t)x % 16 == 0 && (uintptr_t)gamma % 16 == 0 &&
                     (uintptr_t)out % 16 == 0;
  const int words_per_thread = (d / 4 + threads - 1) / threads;
#define GB_LAUNCH(G, O)                                                                                                     \
  do {                                                                                                                      \
    if (words && words_per_thread <= 2)                                                                                     \
      hipLaunchKernelGGL((rmsnorm_words_kernel<G, O, 2>), dim3(m), dim3(threads), 0, stream, x, (const G*)gamma, rows, (O*)out, d, eps); \
    else if (words && words_per_thread <= 4)                                                                                \
      hipLaunchKernelGGL((rmsnorm_words_kernel<G, O, 4>), dim3(m), dim3(threads), 0, stream, x, (const G*)gamma, rows, (O*)out, d, eps); \
    else if (words)                                                                                                         \
      hipLaunchKernelGGL((rmsnorm_words_kernel<G, O, 8>), dim3(m), dim3(threads), 0, stream, x, (const G*)gamma, rows, (O*)out, d, eps); \
    else if (per_thread <= 4)                                                                                               \
      hipLaunchKernelGGL((rmsnorm_kernel<G, O, 4>), dim3(m), dim3(threads), 0, stream, x, (const G*)gamma, rows, (O*)out, d, eps); \
    else                                                                                                                    \
      hipLaunchKernelGGL((rmsnorm_kernel<G, O, 16>), dim3(m), dim3(threads), 0, stream, x, (const G*)gamma, rows, (O*)out, d, eps); \
  } while (0)
  if (gamma_dtype == kF32 && out_dtype == kF32) GB_LAUNCH(float, float);
  else if (gamma_dtype == kF32 && out_dtype == kBF16) GB_LAUNCH(float, bf16);
  else if (gamma_dtype == kBF16 && out_dtype == kF32) GB_LAUNCH(bf16, float);
  else if (gamma_dtype == kBF16 && out_dtype == kBF16) GB_LAUNCH(bf16, bf16);
  else return fail("rmsnorm: unknown dtypes gamma=%d out=%d", gamma_dtype, out_dtype);
#undef GB_LAUNCH
  return launched("rmsnorm");
}

// -------------------------------------------------------------------- rotary table
// angle = f32(pos) * inv[i] as a 32-bit product; sin and cos of it evaluated in 64-bit and
// rounded to 32-bit (model.rs:105-109).  inv comes from the host, computed as the reference does.
__global__ void rope_table_kernel(const int32_t* __restrict__ pos, const float* __restrict__ inv,
                                  float* __restrict__ cosv, float* __restrict__ sinv, int n, int half) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= n * half) return;
  const int t = idx / half, i = idx % half;
  const float a = __fmul_rn((float)pos[t], inv[i]);
  cosv[idx] = (float)cos((double)a);
  sinv[idx] = (float)sin((double)a);
}

extern "C" int gb_rope_table(const int32_t* pos, const float* inv, float* cosv, float* sinv, int n, int half,
                             hipStream_t stream) {
  GB_REQUIRE(n >= 0 && half > 0, "rope_table: bad sizes n=%d half=%d", n, half);
  if (n == 0) return 0;
  const int total = n * half;
  hipLaunchKernelGGL(rope_table_kernel, dim3((total + 255) / 256), dim3(256), 0, stream, pos, inv, cosv, sinv, n, half);
  return launched("rope_table");
}

// ------------------------------------------------- rotation and cache write, fused
// For token t: every query head and key head is rotated in half-split pairs (i, i + hd/2):
//   x0' = x0 c - x1 s ; x1' = x1 c + x0 s                              (model.rs:110-113)
// queries are rotated in place inside the stacked qkv row; rotated keys and plain values go to
// the pages at slot[t] (model.rs:273-275).  Key pages are [page][kv head][hd / piece][slot in page][piece]
// (see key_piece()); value pages are transposed, [page][kv head][hd][slot in page], so that the attention
// kernels find consecutive keys of one value dimension side by side (the matrix cores' operand layout).
// With slots == nullptr nothing is stored (a layer that reads another layer's cache).
// With nkv == 0 the row holds queries only.
template <typename T>
__global__ void rope_store_scalar_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ cosv,
                                  const float* __restrict__ sinv, const int32_t* __restrict__ slots,
                                  T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int hd,
                                  int page_size, int rotate) {
  const int t = blockIdx.x;
  const int half = hd / 2;
  T* row = qkv + (size_t)t * row_stride;
  const float* c = cosv + (size_t)t * half;
  const float* s = sinv + (size_t)t * half;
  const int slot = slots ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const int piece = key_piece(hd);
  // queries, then keys: (nh + nkv) heads of `half` pairs
  const int pairs = (nh + nkv) * half;
  // eight pairs a thread at a time: all loads first, so that they are in flight together (the
  // stores into the row would otherwise order every later load behind them)
  constexpr int B = 8;
  for (int base = threadIdx.x; base < pairs; base += blockDim.x * B) {
    float x0[B], x1[B], cc[B], sn[B];
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int p = base + j * blockDim.x;
      if (p < pairs) {
        const int head = p / half, i = p % half;
        const T* h = row + (size_t)head * hd;
        x0[j] = to_f(h[i]);
        x1[j] = to_f(h[i + half]);
        cc[j] = rotate ? c[i] : 1.f;
        sn[j] = rotate ? s[i] : 0.f;
      }
    }
#pragma unroll
    for (int j = 0; j < B; ++j) {
      const int p = base + j * blockDim.x;
      if (p < pairs) {
        const int head = p / half, i = p % half;
        T* h = row + (size_t)head * hd;
        const T y0 = from_f<T>(rotate ? x0[j] * cc[j] - x1[j] * sn[j] : x0[j]);
        const T y1 = from_f<T>(rotate ? x1[j] * cc[j] + x0[j] * sn[j] : x1[j]);
        h[i] = y0;  // rotated keys stay in the row too: parts may read them back
        h[i + half] = y1;
        if (head >= nh && slot >= 0) {
          T* dst = k_pages + ((size_t)page * nkv + (head - nh)) * page_size * hd;
          dst[key_offset(off, i, page_size, piece)] = y0;
          dst[key_offset(off, i + half, page_size, piece)] = y1;
        }
      }
    }
  }
  if (slot >= 0) {
    const T* v = row + (size_t)(nh + nkv) * hd;
    for (int e = threadIdx.x; e < nkv * hd; e += blockDim.x) {
      const int kvh = e / hd, i = e % hd;
      v_pages[(((size_t)page * nkv + kvh) * hd + i) * page_size + off] = v[e];
    }
  }
}

// The same for head sizes that are a multiple of 4 and rows aligned to two elements: grid (tokens,
// groups of heads), 16 lanes a head, a lane takes two neighbouring pairs as two-element words.  Every
// lane's loads are independent of every store, so one round trip to memory covers a token, and few
// tokens (decoding) still spread over many waves.  A "unit" is a query head, a key head or a value head
// in the order of the row.
template <typename T>
struct Pair {
  T a, b;
};

template <typename T>
__global__ void rope_store_kernel(T* __restrict__ qkv, int row_stride, const float* __restrict__ cosv,
                                  const float* __restrict__ sinv, const int32_t* __restrict__ slots,
                                  T* __restrict__ k_pages, T* __restrict__ v_pages, int nh, int nkv, int hd,
                                  int page_size, int rotate, int v_rows) {
  using P = Pair<T>;
  const int t = blockIdx.x;
  const int half = hd / 2;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int unit = (blockIdx.y * (blockDim.x >> 6) + wave) * 4 + (lane >> 4);
  const int units = nh + nkv + ((slots && t < v_rows) ? nkv : 0);  // rows from v_rows on: values are stored by tiles
  if (unit >= units) return;
  T* head = qkv + (size_t)t * row_stride + (size_t)unit * hd;
  const bool is_v = unit >= nh + nkv, is_k = unit >= nh && !is_v;
  const int slot = (slots && unit >= nh) ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const int piece = key_piece(hd);
  for (int j = (lane & 15) * 2; j < half; j += 32) {
    const P x0 = *reinterpret_cast<const P*>(head + j), x1 = *reinterpret_cast<const P*>(head + half + j);
    P y0 = x0, y1 = x1;
    if (!is_v && rotate) {
      const float2 c = *reinterpret_cast<const float2*>(cosv + (size_t)t * half + j);
      const float2 sn = *reinterpret_cast<const float2*>(sinv + (size_t)t * half + j);
      y0.a = from_f<T>(to_f(x0.a) * c.x - to_f(x1.a) * sn.x);
      y0.b = from_f<T>(to_f(x0.b) * c.y - to_f(x1.b) * sn.y);
      y1.a = from_f<T>(to_f(x1.a) * c.x + to_f(x0.a) * sn.x);
      y1.b = from_f<T>(to_f(x1.b) * c.y + to_f(x0.b) * sn.y);
      *reinterpret_cast<P*>(head + j) = y0;  // rotated keys stay in the row too: parts may read them back
      *reinterpret_cast<P*>(head + half + j) = y1;
    }
    if (slot < 0) continue;
    if (is_k) {
      // j is even and the pieces hold 4 or 8 elements here: a pair stays inside its piece
      T* dst = k_pages + ((size_t)page * nkv + (unit - nh)) * page_size * hd;
      *reinterpret_cast<P*>(dst + key_offset(off, j, page_size, piece)) = y0;
      *reinterpret_cast<P*>(dst + key_offset(off, half + j, page_size, piece)) = y1;
    } else if (is_v) {
      T* dst = v_pages + ((size_t)page * nkv + (unit - nh - nkv)) * hd * page_size + off;
      dst[(size_t)j * page_size] = x0.a;
      dst[(size_t)(j + 1) * page_size] = x0.b;
      dst[(size_t)(half + j) * page_size] = x1.a;
      dst[(size_t)(half + j + 1) * page_size] = x1.b;
    }
  }
}

// The same for head sizes that are a multiple of 16, bfloat16, with 16-byte aligned rows: a lane takes a whole
// piece of 8 dimensions and its partner piece hd/2 further on as 16-byte words, so that a key's pieces go to
// their places in the page (key_piece()) in one store each.  hd / 16 lanes a head.
__device__ __forceinline__ void rope_store_pieces(int t, int idx, bf16* __restrict__ qkv, int row_stride,
                                                  const float* __restrict__ cosv, const float* __restrict__ sinv,
                                                  const int32_t* __restrict__ slots, bf16* __restrict__ k_pages,
                                                  bf16* __restrict__ v_pages, int nh, int nkv, int hd, int page_size,
                                                  int rotate, int v_rows) {
  const int half = hd / 2, lanes = half / 8;  // lanes a head
  const int unit = idx / lanes, j = (idx % lanes) * 8;
  const int units = nh + nkv + ((slots && t < v_rows) ? nkv : 0);  // rows from v_rows on: values are stored by tiles
  if (unit >= units) return;
  bf16* head = qkv + (size_t)t * row_stride + (size_t)unit * hd;
  const bool is_v = unit >= nh + nkv, is_k = unit >= nh && !is_v;
  const int slot = (slots && unit >= nh) ? slots[t] : -1;
  const int page = slot >= 0 ? slot / page_size : 0, off = slot >= 0 ? slot % page_size : 0;
  const bf16x8 x0 = *reinterpret_cast<const bf16x8*>(head + j), x1 = *reinterpret_cast<const bf16x8*>(head + half + j);
  bf16x8 y0 = x0, y1 = x1;
  if (!is_v && rotate) {
    const float* cr = cosv + (size_t)t * half + j;
    const float* sr = sinv + (size_t)t * half + j;
    const f32x4 c0 = *reinterpret_cast<const f32x4*>(cr), c1 = *reinterpret_cast<const f32x4*>(cr + 4);
    const f32x4 s0 = *reinterpret_cast<const f32x4*>(sr), s1 = *reinterpret_cast<const f32x4*>(sr + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float c = e < 4 ? c0[e] : c1[e - 4], sn = e < 4 ? s0[e] : s1[e - 4];
      const float a = (float)x0[e], b = (float)x1[e];
      y0[e] = (bf16)(a * c - b * sn);
      y1[e] = (bf16)(b * c + a * sn);
    }
    *reinterpret_cast<bf16x8*>(head + j) = y0;  // rotated keys stay in the row too: parts may read them back
    *reinterpret_cast<bf16x8*>(head + half + j) = y1;
  }
  if (slot < 0) return;
  if (is_k) {
    bf16* dst = k_pages + ((size_t)page * nkv + (unit - nh)) * page_size * hd;
    *reinterpret_cast<bf16x8*>(dst + key_offset(off, j, page_size, 8)) = y0;
    *reinterpret_cast<bf16x8*>(dst + key_offset(off, half + j, page_size, 8)) = y1;
  } else if (is_v) {
    bf16* dst = v_pages + ((size_t)page * nkv + (unit - nh - nkv)) * hd * page_size + off;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      dst[(size_t)(j + e) * page_size] = x0[e];
      dst[(size_t)(half + j + e) * page_size] = x1[e];
    }
  }
}

__global__ void rope_store_pieces_kernel(bf16* __restrict__ qkv, int row_stride, const float* __restrict__ cosv,
                                         const float* __restrict__ sinv, const int32_t* __restrict__ slots,
                                         bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int nh, int nkv, int hd,
                                         int page_size, int rotate, int v_rows) {
  // The chip deals workgroups round its 8 dies by their number, and each die has a second-level cache of its own: a
  // die takes a run of neighbouring tokens, whose 16-byte pieces lie side by side in a key page, so that the cache
  // writes back whole lines
  int t = blockIdx.x;
  if (gridDim.x % 8 == 0) t = (t % 8) * (gridDim.x / 8) + t / 8;
  rope_store_pieces(t, blockIdx.y * blockDim.x + threadIdx.x, qkv, row_stride, cosv, sinv, slots, k_pages, v_pages, nh,
                    nkv, hd, page_size, rotate, v_rows);
}

// Values of prompt portions, sixteen positions at a time: the transposed page holds the sixteen slots
// of one dimension side by side, so a tile of 16 tokens x hd is turned in LDS and written as whole
// 16-byte words instead of two bytes at a time.  grid (groups of 16 positions, kv heads, requests
// from seq_base on); request s has q_len[s] rows from row q_start[s] on, the first at position pos0[s].
template <typename T>
__device__ __forceinline__ void store_values_tile(int group, int kvh, int seq, T* tile, const T* __restrict__ qkv,
                                                  int row_stride, const int32_t* __restrict__ slots, T* __restrict__ v_pages,
                                                  const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                                  const int32_t* __restrict__ pos0, int nh, int nkv, int hd, int page_size) {
  const int ld = hd + 2;  // tile: [16][hd + 2]
  const int first = pos0[seq], n = q_len[seq];
  const int p_lo = (first / 16 + group) * 16;  // the group's first position
  const int j_lo = p_lo - first;                     // its token index in the portion (may be negative)
  if (j_lo >= n) return;
  const int row0 = q_start[seq];
  const int chunks = hd / 8;
  for (int idx = threadIdx.x; idx < 16 * chunks; idx += blockDim.x) {
    const int i = idx / chunks, ch = idx % chunks, j = j_lo + i;
    if (j < 0 || j >= n) continue;
    const T* src = qkv + (size_t)(row0 + j) * row_stride + (size_t)(nh + nkv + kvh) * hd + ch * 8;
    alignas(16) T got[8];
    *reinterpret_cast<uint4*>(got) = *reinterpret_cast<const uint4*>(src);
    if (sizeof(T) == 4) *reinterpret_cast<uint4*>(got + 4) = *reinterpret_cast<const uint4*>(src + 4);
#pragma unroll
    for (int e = 0; e < 8; ++e) tile[i * ld + ch * 8 + e] = got[e];
  }
  __syncthreads();
  // the page and the first slot of the group, from any token of it that exists
  const int j_any = max(j_lo, 0);
  const int slot_any = slots[row0 + j_any];
  const int page = slot_any / page_size, off0 = slot_any % page_size - (j_any - j_lo);
  T* dst_page = v_pages + ((size_t)page * nkv + kvh) * hd * page_size + off0;
  for (int idx = threadIdx.x; idx < 2 * hd; idx += blockDim.x) {
    const int d = idx / 2, h8 = idx % 2;
    T* dst = dst_page + (size_t)d * page_size + 8 * h8;
    const int i0 = 8 * h8;
    if (j_lo + i0 >= 0 && j_lo + i0 + 8 <= n) {
      alignas(16) T word[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) word[e] = tile[(i0 + e) * ld + d];
      if (sizeof(T) == 2) {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(word);
      } else {
        *reinterpret_cast<uint4*>(dst) = *reinterpret_cast<const uint4*>(word);
        *reinterpret_cast<uint4*>(dst + 4) = *reinterpret_cast<const uint4*>(word + 4);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = j_lo + i0 + e;
        if (j >= 0 && j < n) dst[e] = tile[(i0 + e) * ld + d];
      }
    }
  }
}

template <typename T>
__global__ void store_values_kernel(const T* __restrict__ qkv, int row_stride, const int32_t* __restrict__ slots,
                                    T* __restrict__ v_pages, const int32_t* __restrict__ q_start,
                                    const int32_t* __restrict__ q_len, const int32_t* __restrict__ pos0, int seq_base,
                                    int nh, int nkv, int hd, int page_size) {
  extern __shared__ unsigned char tile_bytes[];
  store_values_tile<T>(blockIdx.x, blockIdx.y, seq_base + blockIdx.z, reinterpret_cast<T*>(tile_bytes), qkv, row_stride, slots,
                       v_pages, q_start, q_len, pos0, nh, nkv, hd, page_size);
}

// Both at once for bfloat16 steps with prompt portions: the first `rope_blocks` workgroups rotate and write keys
// (and the values of single-token rows), the rest turn the portions' values tile by tile.  The two have nothing to
// wait for in each other, and one launch costs a step of some hundred rows less than two.
__global__ void rope_and_values_kernel(bf16* __restrict__ qkv, int row_stride, const float* __restrict__ cosv,
                                       const float* __restrict__ sinv, const int32_t* __restrict__ slots,
                                       bf16* __restrict__ k_pages, bf16* __restrict__ v_pages, int nh, int nkv, int hd,
                                       int page_size, int rotate, int v_rows, int rope_blocks, int rope_y,
                                       const int32_t* __restrict__ q_start, const int32_t* __restrict__ q_len,
                                       const int32_t* __restrict__ pos0, int seq_base, int groups) {
  extern __shared__ unsigned char tile_bytes[];
  const int b = blockIdx.x;
  if (b < rope_blocks) {
    // a die (workgroups b, b + 8, ...) takes a run of neighbouring tokens, as in the kernel above
    const int r = rope_blocks % 8 == 0 ? (b % 8) * (rope_blocks / 8) + b / 8 : b;
    rope_store_pieces(r / rope_y, (r % rope_y) * blockDim.x + threadIdx.x, qkv, row_stride, cosv, sinv, slots, k_pages, v_pages,
                      nh, nkv, hd, page_size, rotate, v_rows);
    return;
  }
  const int v = b - rope_blocks;
  store_values_tile<bf16>(v % groups, v / groups % nkv, seq_base + v / (groups * nkv), reinterpret_cast<bf16*>(tile_bytes), qkv,
                          row_stride, slots, v_pages, q_start, q_len, pos0, nh, nkv, hd, page_size);
}

// Rows v_rows .. n-1 are prompt portions described by q_start, q_len and pos0 of requests seq_base ..
// seq_base + n_seqs - 1 (the longest has max_q_len rows): their values are stored tile by tile.  With
// v_rows == n there are none.
extern "C" int gb_rope_store(void* qkv, int dtype, int row_stride, const float* cosv, const float* sinv,
                             const int32_t* slots, void* k_pages, void* v_pages, int n, int nh, int nkv, int hd,
                             int page_size, int rotate, int v_rows, const int32_t* q_start, const int32_t* q_len,
                             const int32_t* pos0, int seq_base, int n_seqs, int max_q_len, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh >= 0 && nkv >= 0 && hd > 0 && hd % 2 == 0, "rope_store: bad sizes n=%d nh=%d nkv=%d hd=%d", n, nh, nkv, hd);
  GB_REQUIRE(row_stride >= (nh + 2 * nkv) * hd || (slots == nullptr && row_stride >= (nh + nkv) * hd),
             "rope_store: row stride %d is shorter than the stacked heads", row_stride);
  GB_REQUIRE(slots == nullptr || (k_pages && v_pages && page_size > 0), "rope_store: slots given without pages");
  GB_REQUIRE(!rotate || (cosv && sinv), "rope_store: rotation asked without a table");
  if (n == 0) return 0;
  // the tile kernel takes pages of a multiple of 16 slots, head sizes of a multiple of 8 and aligned rows
  const bool tiles = slots && v_rows < n && n_seqs > 0 && q_start && q_len && pos0 && page_size % 16 == 0 && hd % 8 == 0 &&
                     (uintptr_t)v_pages % 16 == 0 && (uintptr_t)qkv % 16 == 0 && row_stride % 8 == 0;
  if (!tiles) v_rows = n;
  const bool pairs_of_two = hd % 4 == 0 && row_stride % 2 == 0 && (uintptr_t)qkv % 8 == 0 && (uintptr_t)k_pages % 8 == 0 &&
                            (!rotate || ((uintptr_t)cosv % 8 == 0 && (uintptr_t)sinv % 8 == 0));
  const bool pieces = dtype == kBF16 && hd % 16 == 0 && row_stride % 8 == 0 && (uintptr_t)qkv % 16 == 0 &&
                      (uintptr_t)k_pages % 16 == 0 && (!rotate || ((uintptr_t)cosv % 16 == 0 && (uintptr_t)sinv % 16 == 0));
  // one launch for both while the launch it saves weighs more than the value tiles' larger workgroups in it cost
  // (2,048 tokens: 22.6 us in one launch, 13.9 + 6.9 in two; 128 tokens: 4.7 against 3.6 + 3.7)
  if (tiles && pieces && n <= 1024) {
    const int units = nh + 2 * nkv, lanes = units * (hd / 16);
    const int threads = lanes >= 256 ? 256 : 64;
    const int rope_y = (lanes + threads - 1) / threads, groups = (max_q_len + 15) / 16 + 1;
    const long long blocks = (long long)n * rope_y + (long long)groups * nkv * n_seqs;
    GB_REQUIRE(blocks < (1ll << 31), "rope_store: %lld workgroups are too many for one launch", blocks);
    hipLaunchKernelGGL(rope_and_values_kernel, dim3((unsigned)blocks), dim3(threads), 16 * (hd + 2) * sizeof(bf16), stream,
                       (bf16*)qkv, row_stride, cosv, sinv, slots, (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, page_size, rotate,
                       v_rows, n * rope_y, rope_y, q_start, q_len, pos0, seq_base, groups);
    return launched("rope_store (with the portions' values)");
  }
  if (tiles) {
    const dim3 grid((max_q_len + 15) / 16 + 1, nkv, n_seqs);
    GB_REQUIRE(nkv <= 65535 && n_seqs <= 65535, "rope_store: too many kv heads or requests for one launch");
    const int threads = 2 * hd >= 256 ? 256 : 128;
    if (dtype == kF32)
      hipLaunchKernelGGL(store_values_kernel<float>, grid, dim3(threads), 16 * (hd + 2) * sizeof(float), stream,
                         (const float*)qkv, row_stride, slots, (float*)v_pages, q_start, q_len, pos0, seq_base, nh, nkv, hd,
                         page_size);
    else if (dtype == kBF16)
      hipLaunchKernelGGL(store_values_kernel<bf16>, grid, dim3(threads), 16 * (hd + 2) * sizeof(bf16), stream,
                         (const bf16*)qkv, row_stride, slots, (bf16*)v_pages, q_start, q_len, pos0, seq_base, nh, nkv, hd,
                         page_size);
    else
      return fail("rope_store: unknown dtype %d", dtype);
    if (int rc = launched("rope_store (values)")) return rc;
  }
  if (pieces) {
    const int units = nh + nkv + (slots ? nkv : 0), lanes = units * (hd / 16);
    const int threads = lanes >= 256 ? 256 : 64;
    const dim3 grid(n, (lanes + threads - 1) / threads);
    GB_REQUIRE(grid.y <= 65535, "rope_store: %d heads are too many for one launch", units);
    hipLaunchKernelGGL(rope_store_pieces_kernel, grid, dim3(threads), 0, stream, (bf16*)qkv, row_stride, cosv, sinv, slots,
                       (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, page_size, rotate, v_rows);
    return launched("rope_store");
  }
  if (pairs_of_two) {
    const int units = nh + nkv + (slots ? nkv : 0);
    const int threads = n <= 64 ? 64 : 256;  // few tokens: more, smaller workgroups
    const dim3 grid(n, (units + threads / 16 - 1) / (threads / 16));
    GB_REQUIRE(grid.y <= 65535, "rope_store: %d heads are too many for one launch", units);
    if (dtype == kF32)
      hipLaunchKernelGGL(rope_store_kernel<float>, grid, dim3(threads), 0, stream, (float*)qkv, row_stride, cosv, sinv, slots,
                         (float*)k_pages, (float*)v_pages, nh, nkv, hd, page_size, rotate, v_rows);
    else if (dtype == kBF16)
      hipLaunchKernelGGL(rope_store_kernel<bf16>, grid, dim3(threads), 0, stream, (bf16*)qkv, row_stride, cosv, sinv, slots,
                         (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, page_size, rotate, v_rows);
    else
      return fail("rope_store: unknown dtype %d", dtype);
    return launched("rope_store");
  }
  const int threads = (nh + nkv) * hd / 2 >= 256 ? 256 : 64;
  if (dtype == kF32)
    hipLaunchKernelGGL(rope_store_scalar_kernel<float>, dim3(n), dim3(threads), 0, stream, (float*)qkv, row_stride, cosv, sinv,
                       slots, (float*)k_pages, (float*)v_pages, nh, nkv, hd, page_size, rotate);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(rope_store_scalar_kernel<bf16>, dim3(n), dim3(threads), 0, stream, (bf16*)qkv, row_stride, cosv, sinv,
                       slots, (bf16*)k_pages, (bf16*)v_pages, nh, nkv, hd, page_size, rotate);
  else
    return fail("rope_store: unknown dtype %d", dtype);
  return launched("rope_store");
}

// ------------------------------------------------------------------- SiLU-multiply
// act = g / (1 + exp(-g)) * u, gate in the first I columns, up in the last I (model.rs:336-340)
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ act, int n, int inter) {
  const size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= (size_t)n * inter) return;
  const size_t t = idx / inter, c = idx % inter;
  const float g = to_f(gu[t * 2 * inter + c]);
  const float u = to_f(gu[t * 2 * inter + inter + c]);
  act[idx] = from_f<T>(g / (1.0f + expf(-g)) * u);
}

extern "C" int gb_silu_mul(const void* gu, void* act, int dtype, int n, int inter, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && inter > 0, "silu_mul: bad sizes n=%d inter=%d", n, inter);
  if (n == 0) return 0;
  const size_t total = (size_t)n * inter;
  const dim3 grid((unsigned)((total + 255) / 256));
  if (dtype == kF32)
    hipLaunchKernelGGL(silu_mul_kernel<float>, grid, dim3(256), 0, stream, (const float*)gu, (float*)act, n, inter);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16>, grid, dim3(256), 0, stream, (const bf16*)gu, (bf16*)act, n, inter);
  else
    return fail("silu_mul: unknown dtype %d", dtype);
  return launched("silu_mul");
}

// ---------------------------------------------------------------------- row copies
// base is [rows][row_bytes]; copies row src[i] onto row dst[i] (copy-on-write of a page in one
// layer's pool, kv.rs:189-196, and copies of state slots).  row_bytes is a multiple of 4.
__global__ void copy_rows_kernel(uint32_t* __restrict__ base, size_t row_words, const int32_t* __restrict__ src,
                                 const int32_t* __restrict__ dst) {
  const uint32_t* s = base + (size_t)src[blockIdx.x] * row_words;
  uint32_t* d = base + (size_t)dst[blockIdx.x] * row_words;
  for (size_t w = threadIdx.x; w < row_words; w += blockDim.x) d[w] = s[w];
}

extern "C" int gb_copy_rows(void* base, long long row_bytes, const int32_t* src, const int32_t* dst, int count,
                            hipStream_t stream) {
  GB_REQUIRE(row_bytes > 0 && row_bytes % 4 == 0, "copy_rows: row of %lld bytes is not a multiple of 4", row_bytes);
  if (count <= 0) return 0;
  hipLaunchKernelGGL(copy_rows_kernel, dim3(count), dim3(256), 0, stream, (uint32_t*)base, (size_t)(row_bytes / 4), src, dst);
  return launched("copy_rows");
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_embed)
GB_TAPED(gb_rmsnorm)
GB_TAPED(gb_rope_table)
GB_TAPED(gb_rope_store)
GB_TAPED(gb_silu_mul)
GB_TAPED(gb_copy_rows)
