// Plain paged attention, one block per (token, query head), any head size up to 256, any
// number of heads and groups, 32-bit or bfloat16 storage with 32-bit arithmetic throughout.
// It is the attention of the true 32-bit path (prompt portions and decoded tokens alike) and
// the twin that the tuned bfloat16 kernels are checked against.
//
// Token t of request s at position p reads keys lo..p of its own request through the block
// table, lo = 0 or p - window + 1 (crates/glassbox-core/src/model.rs:285-312):
//   score = dot(q, k) * scale ; prob = softmax(score) ; out = sum prob * v
// Keys are taken in chunks of 256 in ascending position with a running maximum and sum, so
// the order of every addition depends on the position alone, not on the batch.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int kChunk = 256;

template <typename T>
__global__ __launch_bounds__(kChunk) void attention_plain_kernel(
    const T* __restrict__ q, int q_stride, T* __restrict__ out, int out_stride, const int32_t* __restrict__ positions,
    const int32_t* __restrict__ tok_seq, const int32_t* __restrict__ tables, int table_stride,
    const T* __restrict__ k_pages, const T* __restrict__ v_pages, int nh, int nkv, int hd, int page_size, float scale,
    int window) {
  extern __shared__ float smem[];
  float* qs = smem;              // [hd]
  float* es = smem + hd;         // [kChunk]
  float* scratch = es + kChunk;  // [17]
  const int t = blockIdx.x / nh, h = blockIdx.x % nh;
  const int kvh = h / (nh / nkv);
  const int pos = positions[t];
  const int32_t* table = tables + (size_t)tok_seq[t] * table_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int tid = threadIdx.x;
  const int piece = key_piece(hd);

  for (int d = tid; d < hd; d += kChunk) qs[d] = to_f(q[(size_t)t * q_stride + (size_t)h * hd + d]);
  __syncthreads();

  float m = -INFINITY, l = 0.f, acc = 0.f;  // acc: output dimension `tid` (tid < hd)
  for (int c0 = lo; c0 <= pos; c0 += kChunk) {
    const int p = c0 + tid;
    float s = -INFINITY;
    if (p <= pos) {
      const int page = table[p / page_size];
      const T* kb = k_pages + ((size_t)page * nkv + kvh) * page_size * hd;  // pieces of the head size, see key_piece()
      float dot = 0.f;
      for (int d0 = 0; d0 < hd; d0 += piece) {
        const T* kr = kb + key_offset(p % page_size, d0, page_size, piece);
        for (int e = 0; e < piece; ++e) dot = fmaf(qs[d0 + e], to_f(kr[e]), dot);
      }
      s = dot * scale;
    }
    const float cm = block_max(s, scratch);
    const float m_new = fmaxf(m, cm);
    const float e = p <= pos ? expf(s - m_new) : 0.f;
    es[tid] = e;
    const float csum = block_sum(e, scratch);  // also orders the writes of es before the reads below
    const float rescale = expf(m - m_new);     // 0 on the first chunk (m = -inf)
    l = l * rescale + csum;
    acc *= rescale;
    if (tid < hd) {
      const int cnt = min(kChunk, pos - c0 + 1);
      for (int j = 0; j < cnt; ++j) {
        const int pj = c0 + j;
        const int page = table[pj / page_size];
        acc = fmaf(es[j], to_f(v_pages[(((size_t)page * nkv + kvh) * hd + tid) * page_size + pj % page_size]), acc);
      }
    }
    m = m_new;
    __syncthreads();
  }
  if (tid < hd) out[(size_t)t * out_stride + (size_t)h * hd + tid] = from_f<T>(acc / l);
}

}  // namespace

extern "C" int gb_attention_plain(const void* q, int q_stride, void* out, int out_stride, int dtype,
                                  const int32_t* positions, const int32_t* tok_seq, const int32_t* tables,
                                  int table_stride, const void* k_pages, const void* v_pages, int n, int nh, int nkv,
                                  int hd, int page_size, float scale, int window, hipStream_t stream) {
  GB_REQUIRE(n >= 0 && nh > 0 && nkv > 0 && hd > 0, "attention_plain: bad sizes n=%d nh=%d nkv=%d hd=%d", n, nh, nkv, hd);
  GB_REQUIRE(nh % nkv == 0, "attention_plain: %d query heads are not a multiple of %d key heads", nh, nkv);
  GB_REQUIRE(hd <= kChunk, "attention_plain: head size %d is above the supported 256", hd);
  GB_REQUIRE(q_stride >= nh * hd && out_stride >= nh * hd, "attention_plain: row strides shorter than the heads");
  GB_REQUIRE(page_size > 0 && table_stride > 0 && window >= 0, "attention_plain: bad page size, table stride or window");
  GB_REQUIRE((long long)n * nh < (1ll << 31), "attention_plain: too many (token, head) pairs");
  if (n == 0) return 0;
  const size_t smem = sizeof(float) * (hd + kChunk + 17);
  const dim3 grid((unsigned)(n * nh));
  if (dtype == kF32)
    hipLaunchKernelGGL(attention_plain_kernel<float>, grid, dim3(kChunk), smem, stream, (const float*)q, q_stride,
                       (float*)out, out_stride, positions, tok_seq, tables, table_stride, (const float*)k_pages,
                       (const float*)v_pages, nh, nkv, hd, page_size, scale, window);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(attention_plain_kernel<bf16>, grid, dim3(kChunk), smem, stream, (const bf16*)q, q_stride,
                       (bf16*)out, out_stride, positions, tok_seq, tables, table_stride, (const bf16*)k_pages,
                       (const bf16*)v_pages, nh, nkv, hd, page_size, scale, window);
  else
    return fail("attention_plain: unknown dtype %d", dtype);
  return launched("attention_plain");
}

// the launches of a layer can be recorded and made again for the layers like it (common.h)
GB_TAPED(gb_attention_plain)
