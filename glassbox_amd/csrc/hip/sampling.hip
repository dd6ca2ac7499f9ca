// Turning rows of logits into tokens on the device: argmax, the repetition penalty, and the
// reference's sampler with all of its filters (crates/glassbox-core/src/sampler.rs:97-164).
//
// The reference sorts the candidates by descending logit and then works on prefixes of that
// order: top-k keeps the first k, min-p the ones at least p_max*min_p, top-p the shortest prefix
// whose probability reaches top_p, and the draw walks the same order until the running
// probability passes a uniform number.  Nothing here sorts.  The order is a 52-bit key per
// token (the logit's bits made monotone, then the token id, so equal logits go by id), and
// "the first element where the running weight crosses a target" is found by a radix search
// over that key, 4 bits a pass, with per-thread bins in LDS and fixed-order reductions so that
// the result does not depend on timing.  The uniform number comes from the host, which owns
// each request's generator.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int TPB = 256;
constexpr int BINS = 16;
constexpr int IDX_BITS = 20;   // vocabulary up to 2^20
constexpr int KEY_BITS = 32 + IDX_BITS;

__device__ __forceinline__ uint32_t ordered_bits(float v) {
  const uint32_t u = __float_as_uint(v);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);  // larger float -> larger unsigned
}
// larger composite = earlier in the reference's order (larger logit first, then smaller id)
__device__ __forceinline__ uint64_t composite(float v, int idx) {
  return ((uint64_t)ordered_bits(v) << IDX_BITS) | (uint64_t)(((1u << IDX_BITS) - 1u) - (uint32_t)idx);
}

// ---------------------------------------------------------------------------- argmax
// first maximum wins (sampler.rs:49-57) = the largest composite key
constexpr int ARGMAX_TPB = 1024;
__global__ __launch_bounds__(ARGMAX_TPB) void argmax_kernel(const float* __restrict__ logits, int32_t* __restrict__ out, int V) {
  __shared__ uint64_t best[ARGMAX_TPB / kWave];
  const float* row = logits + (size_t)blockIdx.x * V;
  uint64_t b = 0;
  // four loads in flight per thread
  for (int i0 = threadIdx.x; i0 < V; i0 += 4 * ARGMAX_TPB) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i0 + j * ARGMAX_TPB < V ? row[i0 + j * ARGMAX_TPB] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j * ARGMAX_TPB;
      const uint64_t c = i < V ? composite(v[j], i) : 0;
      b = c > b ? c : b;
    }
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const uint64_t other = __shfl_xor(b, o, kWave);
    b = other > b ? other : b;
  }
  if (threadIdx.x % kWave == 0) best[threadIdx.x / kWave] = b;
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < ARGMAX_TPB / kWave; ++w) b = best[w] > b ? best[w] : b;
    out[blockIdx.x] = (int32_t)(((1u << IDX_BITS) - 1u) - (uint32_t)(b & ((1u << IDX_BITS) - 1u)));
  }
}

// -------------------------------------------------------------------------- penalty
// For a token that occurs `count` times in the context: count times v = v > 0 ? v / pen : v * pen
// (sampler.rs:100-108).  One thread per (row, distinct token) pair, prepared by the host.
__global__ void penalize_kernel(float* __restrict__ logits, int V, const int32_t* __restrict__ rows,
                                const int32_t* __restrict__ tokens, const int32_t* __restrict__ counts,
                                const float* __restrict__ penalties, int pairs) {
  const int p = blockIdx.x * blockDim.x + threadIdx.x;
  if (p >= pairs) return;
  const int tok = tokens[p];
  if (tok < 0 || tok >= V) return;
  float* v = logits + (size_t)rows[p] * V + tok;
  const float pen = penalties[p];
  float x = *v;
  for (int c = 0; c < counts[p]; ++c) x = x > 0.f ? x / pen : x * pen;
  *v = x;
}

// --------------------------------------------------------------------------- sampler
struct Row {
  const float* logits;
  int V;
  float temperature;
  float mx;          // max of logit / T
  float S;           // sum of exp over the top-k candidates
  float minp_floor;  // probabilities below it are dropped; 0 = none
  uint64_t cut;      // members have composite >= cut
};

__device__ __forceinline__ float scaled(const Row& r, int i) { return r.logits[i] / r.temperature; }
__device__ __forceinline__ float prob(const Row& r, float l) { return expf(l - r.mx) / r.S; }
__device__ __forceinline__ bool member(const Row& r, float l, int i) {
  if (composite(l, i) < r.cut) return false;
  return r.minp_floor <= 0.f || prob(r, l) >= r.minp_floor;
}

struct Shared {
  float w[BINS][TPB];
  int c[BINS][TPB];
  float pw[BINS][TPB / kWave];
  int pc[BINS][TPB / kWave];
  uint64_t prefix;
  float cum;
  int done;       // 1: one element is left under the prefix
  int fallback;
  int shift;
  float fscratch[17];
  int iscratch[17];
  uint64_t found;
};

__device__ __forceinline__ int block_count(int v, Shared& sh) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  __syncthreads();
  if (lane == 0) sh.iscratch[wave] = v;
  __syncthreads();
  if (threadIdx.x == 0) {
    int t = 0;
    for (int w = 0; w < TPB / kWave; ++w) t += sh.iscratch[w];
    sh.iscratch[16] = t;
  }
  __syncthreads();
  return sh.iscratch[16];
}

// Among the members of `r`, in descending key order, the first element at which the running
// weight reaches the target: weight 1 per element (COUNT) or its probability.  STRICT: the
// running weight must exceed the target (the draw's `r < acc`); otherwise reach it (`acc >= top_p`,
// rank k).  If rounding keeps the total below the target, the last member is returned, as the
// reference falls back to the last candidate.  Returns the element's composite key.
template <bool COUNT, bool STRICT>
__device__ uint64_t select(const Row& r, float target, Shared& sh) {
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  if (tid == 0) {
    sh.prefix = 0;
    sh.cum = 0.f;
    sh.done = 0;
    sh.fallback = 0;
  }
  __syncthreads();
  for (int shift = KEY_BITS - 4; shift >= 0; shift -= 4) {
    const uint64_t prefix = sh.prefix;
#pragma unroll
    for (int b = 0; b < BINS; ++b) {
      sh.w[b][tid] = 0.f;
      sh.c[b][tid] = 0;
    }
    for (int i = tid; i < r.V; i += TPB) {
      const float l = scaled(r, i);
      if (!member(r, l, i)) continue;
      const uint64_t c = composite(l, i);
      if ((c >> (shift + 4)) != prefix) continue;
      const int d = (int)((c >> shift) & (BINS - 1));
      sh.w[d][tid] += COUNT ? 1.f : prob(r, l);
      sh.c[d][tid] += 1;
    }
    // per bin: waves reduce their lanes in a fixed butterfly, thread 0 adds the waves in order
#pragma unroll
    for (int b = 0; b < BINS; ++b) {
      float wv = sh.w[b][tid];
      int cv = sh.c[b][tid];
#pragma unroll
      for (int o = kWave / 2; o > 0; o >>= 1) {
        wv += __shfl_xor(wv, o, kWave);
        cv += __shfl_xor(cv, o, kWave);
      }
      if (lane == 0) {
        sh.pw[b][wave] = wv;
        sh.pc[b][wave] = cv;
      }
    }
    __syncthreads();
    if (tid == 0) {
      int pick = -1, lowest = -1;
      float cum = sh.cum;
      for (int b = BINS - 1; b >= 0; --b) {
        float wv = 0.f;
        int cv = 0;
        for (int w = 0; w < TPB / kWave; ++w) {
          wv += sh.pw[b][w];
          cv += sh.pc[b][w];
        }
        if (cv == 0) continue;
        lowest = b;
        sh.pc[b][0] = cv;
        if (!sh.fallback) {
          const float reach = cum + wv;
          if (STRICT ? reach > target : reach >= target) {
            pick = b;
            break;
          }
          cum = reach;
        }
      }
      if (pick < 0) {  // the weights never reach the target: take the last member
        sh.fallback = 1;
        pick = lowest;
      }
      sh.cum = cum;
      sh.prefix = (prefix << 4) | (uint64_t)(pick < 0 ? 0 : pick);
      sh.done = (pick >= 0 && sh.pc[pick][0] == 1) ? 1 : 0;
      sh.shift = shift;
    }
    __syncthreads();
    if (sh.done) break;
  }
  const int shift = sh.shift;
  if (shift == 0 || !sh.done) {
    return sh.prefix;  // every bit decided
  }
  // one member is left under the prefix: find it
  const uint64_t prefix = sh.prefix;
  for (int i = tid; i < r.V; i += TPB) {
    const float l = scaled(r, i);
    if (!member(r, l, i)) continue;
    const uint64_t c = composite(l, i);
    if ((c >> shift) == prefix) sh.found = c;
  }
  __syncthreads();
  return sh.found;
}

__global__ __launch_bounds__(TPB) void sample_kernel(const float* __restrict__ logits, int V,
                                                     const float* __restrict__ temperature, const int32_t* __restrict__ top_k,
                                                     const float* __restrict__ top_p, const float* __restrict__ min_p,
                                                     const float* __restrict__ uniform, int32_t* __restrict__ out_token,
                                                     int32_t* __restrict__ out_candidates) {
  __shared__ Shared sh;
  const int rix = blockIdx.x, tid = threadIdx.x;
  Row r;
  r.logits = logits + (size_t)rix * V;
  r.V = V;
  r.temperature = temperature[rix];
  r.mx = 0.f;
  r.S = 1.f;
  r.minp_floor = 0.f;
  r.cut = 0;
  const uint32_t idx_mask = (1u << IDX_BITS) - 1u;

  // the first maximum: needed by greedy rows and as the softmax's reference point
  const bool greedy = !(r.temperature > 0.f);
  if (greedy) r.temperature = 1.f;
  uint64_t b = 0;
  for (int i = tid; i < V; i += TPB) {
    const uint64_t c = composite(scaled(r, i), i);
    b = c > b ? c : b;
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const uint64_t other = __shfl_xor(b, o, kWave);
    b = other > b ? other : b;
  }
  __shared__ uint64_t wbest[TPB / kWave];
  if (tid % kWave == 0) wbest[tid / kWave] = b;
  __syncthreads();
  b = wbest[0];
  for (int w = 1; w < TPB / kWave; ++w) b = wbest[w] > b ? wbest[w] : b;
  const int best_idx = (int)(idx_mask - (uint32_t)(b & idx_mask));
  if (greedy) {  // sampler.rs:110-112
    if (tid == 0) {
      out_token[rix] = best_idx;
      out_candidates[rix] = 1;
    }
    return;
  }
  r.mx = scaled(r, best_idx);

  // top-k: the k-th element of the order closes the candidate set (sampler.rs:116-117)
  const int k = top_k[rix];
  if (k > 0 && k < V) r.cut = select<true, false>(r, (float)k, sh);
  // softmax over the candidates (sampler.rs:118-126)
  float part = 0.f;
  for (int i = tid; i < V; i += TPB) {
    const float l = scaled(r, i);
    if (composite(l, i) >= r.cut) part += expf(l - r.mx);
  }
  r.S = block_sum(part, sh.fscratch);
  // min-p: drop what lies below p_max * min_p, p_max being the first candidate's (sampler.rs:127-130)
  const float mp = min_p[rix];
  if (mp > 0.f) r.minp_floor = (1.0f / r.S) * mp;
  // top-p: the shortest prefix whose probability reaches top_p (sampler.rs:131-142)
  const float tp = top_p[rix];
  if (tp < 1.f) {
    const uint64_t cut = select<false, false>(r, tp, sh);
    r.cut = cut > r.cut ? cut : r.cut;
  }
  // renormalise over what is left and draw (sampler.rs:143-146,155-163)
  float tpart = 0.f;
  int cpart = 0;
  for (int i = tid; i < V; i += TPB) {
    const float l = scaled(r, i);
    if (member(r, l, i)) {
      tpart += prob(r, l);
      cpart += 1;
    }
  }
  const float total = block_sum(tpart, sh.fscratch);
  const int candidates = block_count(cpart, sh);
  uint64_t chosen = b;  // a single candidate is the first maximum; no draw
  if (candidates > 1) chosen = select<false, true>(r, uniform[rix] * total, sh);
  if (tid == 0) {
    out_token[rix] = (int32_t)(idx_mask - (uint32_t)(chosen & idx_mask));
    out_candidates[rix] = candidates;
  }
}

}  // namespace

extern "C" int gb_argmax(const float* logits, int32_t* out, int rows, int V, hipStream_t stream) {
  GB_REQUIRE(rows >= 0 && V > 0 && V <= (1 << IDX_BITS), "argmax: vocabulary %d is outside 1..%d", V, 1 << IDX_BITS);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(argmax_kernel, dim3(rows), dim3(ARGMAX_TPB), 0, stream, logits, out, V);
  return launched("argmax");
}

extern "C" int gb_penalize(float* logits, int V, const int32_t* rows, const int32_t* tokens, const int32_t* counts,
                           const float* penalties, int pairs, hipStream_t stream) {
  GB_REQUIRE(V > 0 && pairs >= 0, "penalize: bad sizes");
  if (pairs == 0) return 0;
  hipLaunchKernelGGL(penalize_kernel, dim3((pairs + 255) / 256), dim3(256), 0, stream, logits, V, rows, tokens, counts,
                     penalties, pairs);
  return launched("penalize");
}

extern "C" int gb_sample(const float* logits, int rows, int V, const float* temperature, const int32_t* top_k,
                         const float* top_p, const float* min_p, const float* uniform, int32_t* out_token,
                         int32_t* out_candidates, hipStream_t stream) {
  GB_REQUIRE(rows >= 0 && V > 0 && V <= (1 << IDX_BITS), "sample: vocabulary %d is outside 1..%d", V, 1 << IDX_BITS);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(TPB), 0, stream, logits, V, temperature, top_k, top_p, min_p,
                     uniform, out_token, out_candidates);
  return launched("sample");
}
