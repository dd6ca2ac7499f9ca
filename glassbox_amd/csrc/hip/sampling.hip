// Turning rows of logits into tokens on the device: argmax, the repetition penalty, and the
// reference's sampler with all of its filters (crates/glassbox-core/src/sampler.rs:97-164).
//
// The reference sorts the candidates by descending logit and then works on prefixes of that
// order: top-k keeps the first k, min-p the ones at least p_max*min_p, top-p the shortest prefix
// whose probability reaches top_p, and the draw walks the same order until the running
// probability passes a uniform number.  Nothing here sorts.  The order is a 52-bit key per
// token (the logit's bits made monotone, then the token id, so equal logits go by id), and
// "the first element where the running weight crosses a target" is found by a search over
// bins of values and then of keys (see the sampler below), with weights that are whole numbers,
// so that the result does not depend on timing.  The uniform number comes from the host, which
// owns each request's generator.
#include "common.h"

using namespace gb;

GB_DEFINE_LAST_ERROR

namespace {

constexpr int IDX_BITS = 20;   // vocabulary up to 2^20

__device__ __forceinline__ uint32_t ordered_bits(float v) {
  const uint32_t u = v == 0.f ? 0u : __float_as_uint(v);  // -0 and +0 are one value: they go by token id
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
// One workgroup of 1,024 threads a row.  Every filter of the reference keeps a prefix of the descending order, so a
// row's state is one key (`cut`: members have composite >= cut) and the min-p floor, and every question is "the
// first member at which the running weight reaches a target", the weight of a member being 1 (top-k) or its
// probability (top-p, the draw).  Probabilities are carried as whole numbers, exp(l - max) * 2^40 in 64 bits: sums
// of whole numbers do not depend on the order in which the threads add, so bins can be filled with LDS atomics
// and the result still does not depend on timing.
//
// select() finds that member in a few passes over the row (which the second-level cache holds): 2,048 bins that
// divide the members' range of values evenly (so that a row's many middling logits spread over the bins and their
// atomics seldom meet), a scan of the bins from the top for the one in which the target is reached, the smallest
// and largest key in that bin, then 2,048 bins over that range of keys, and so on until a bin is a single key.
constexpr int TPB = 1024;
constexpr int LEVEL_BITS = 11, BINS = 1 << LEVEL_BITS;
constexpr float kWeightOne = 1099511627776.f;  // 2^40: the weight of the row's maximum
typedef unsigned long long u64;

struct Row {
  const float* logits;  // already divided by the temperature
  int V;
  float mx;          // the largest
  float S;           // sum of exp over the top-k candidates
  float minp_floor;  // probabilities below it are dropped; 0 = none
  u64 cut;           // members have composite >= cut
};

__device__ __forceinline__ float prob(const Row& r, float l) { return expf(l - r.mx) / r.S; }
// exp(l - max) in units of 2^-40, by the hardware's exponential: what the sums and targets below are made of
__device__ __forceinline__ u64 weight(const Row& r, float l) { return (u64)(__expf(l - r.mx) * kWeightOne); }
__device__ __forceinline__ bool member(const Row& r, float l, u64 key) {
  if (key < r.cut) return false;
  return r.minp_floor <= 0.f || prob(r, l) >= r.minp_floor;
}

// f(l, i) for every token of the row; four loads in flight a thread, a thread's tokens in ascending order
template <typename F>
__device__ __forceinline__ void for_each(const float* __restrict__ row, int V, F f) {
  for (int i0 = threadIdx.x; i0 < V; i0 += 4 * TPB) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i0 + j * TPB < V ? row[i0 + j * TPB] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j)
      if (i0 + j * TPB < V) f(v[j], i0 + j * TPB);
  }
}

struct Shared {
  unsigned int cnt[BINS];
  u64 w[BINS];
  u64 waves[TPB / kWave], waves2[TPB / kWave];
  u64 cum, lo, hi;
  int pick, last;
};

// Sums of two numbers over the workgroup; every thread gets them.
__device__ __forceinline__ void block_totals(u64& a, u64& b, Shared& sh) {
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    a += __shfl_xor(a, o, kWave);
    b += __shfl_xor(b, o, kWave);
  }
  __syncthreads();
  if (threadIdx.x % kWave == 0) {
    sh.waves[threadIdx.x / kWave] = a;
    sh.waves2[threadIdx.x / kWave] = b;
  }
  __syncthreads();
  a = b = 0;
#pragma unroll
  for (int w = 0; w < TPB / kWave; ++w) {
    a += sh.waves[w];
    b += sh.waves2[w];
  }
  __syncthreads();
}

// What select() is asked for: the first member at which the running weight reaches `need`, or, with need == 0,
// `fraction` of all members' weight (or of `of`, if that is given): reached (top-p: acc >= top_p) or, if `strict`,
// passed (the draw: r < acc).
struct Target {
  u64 need;
  double fraction;
  u64 of;
  bool strict;
};

// The bins hold counts and weights, bin BINS-1 first in the order.  Finds the first bin that holds something and
// in which cum + (weights from the top) reaches `need`; if none does (or an earlier level found none: `fallback`),
// the last bin that holds something, as the reference falls back to its last candidate.  Returns the bin; sh.cum
// becomes cum + the weights above it.  With `t` (the first level) the need is worked out here from the bins' total,
// and total and count of all bins are handed back.
template <bool COUNT>
__device__ int pick_bin(u64& need, bool& fallback, Shared& sh, const Target* t = nullptr, u64* total = nullptr,
                        u64* count = nullptr) {
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  constexpr int PER = BINS / TPB;
  u64 wt[PER], local = 0, members = 0;
  unsigned int cn[PER];
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    const int b = BINS - 1 - (tid * PER + j);
    cn[j] = sh.cnt[b];
    wt[j] = COUNT ? (u64)cn[j] : sh.w[b];
    local += wt[j];
    members += cn[j];
  }
  if (t != nullptr) {
    u64 all = local;
    block_totals(all, members, sh);
    *total = all;
    *count = members;
    need = t->need;
    if (need == 0) {
      const double x = t->fraction * (double)(t->of ? t->of : all);
      need = t->strict ? (u64)floor(x) + 1 : (u64)ceil(x);
    }
  }
  u64 x = local;  // inclusive scan over the threads in order
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const u64 y = __shfl_up(x, o, kWave);
    if (lane >= o) x += y;
  }
  if (tid == 0) {
    sh.pick = BINS;
    sh.last = -1;
  }
  if (lane == kWave - 1) sh.waves[wave] = x;
  __syncthreads();
  u64 above = sh.cum + x - local;
  for (int w = 0; w < wave; ++w) above += sh.waves[w];
  int first = BINS, last = -1;
  u64 run = above;
#pragma unroll
  for (int j = 0; j < PER; ++j) {
    run += wt[j];
    if (cn[j] != 0) {
      last = tid * PER + j;
      if (first == BINS && run >= need) first = tid * PER + j;
    }
  }
  if (first < BINS && !fallback) atomicMin(&sh.pick, first);
  if (last >= 0) atomicMax(&sh.last, last);
  __syncthreads();
  int rank = sh.pick;
  if (rank == BINS) {
    fallback = true;
    rank = sh.last;
  }
  if (rank >= tid * PER && rank < (tid + 1) * PER) {
    u64 c = above;
#pragma unroll
    for (int j = 0; j < PER; ++j)
      if (tid * PER + j < rank) c += wt[j];
    sh.cum = c;
  }
  __syncthreads();
  return BINS - 1 - rank;
}

// Among the members of `r`, in descending key order, the first at which the running weight (1 an element if COUNT,
// else weight()) reaches the target; the last member if the weights never do; 0 if there is no member.  `lowest`: a
// value no member lies below.  Hands back the members' weight and number.
template <bool COUNT>
__device__ u64 select(const Row& r, const Target& target, float lowest, Shared& sh, u64* total, u64* count) {
  const int tid = threadIdx.x;
  bool fallback = false;
  // bins that divide [lowest, max] evenly
  const float scale = r.mx > lowest ? (float)(BINS - 1) / (r.mx - lowest) : 0.f;
  auto value_bin = [&](float l) { return BINS - 1 - min(BINS - 1, max(0, (int)((r.mx - l) * scale))); };
  for (int b = tid; b < BINS; b += TPB) {
    sh.cnt[b] = 0;
    sh.w[b] = 0;
  }
  if (tid == 0) sh.cum = 0;
  __syncthreads();
  for_each(r.logits, r.V, [&](float l, int i) {
    if (!member(r, l, composite(l, i))) return;
    const int b = value_bin(l);
    atomicAdd(&sh.cnt[b], 1u);
    if (!COUNT) atomicAdd(&sh.w[b], weight(r, l));
  });
  __syncthreads();
  u64 need;
  const int vbin = pick_bin<COUNT>(need, fallback, sh, &target, total, count);
  if (*count == 0) return 0;
  // the smallest and largest key in that bin
  if (tid == 0) {
    sh.lo = ~0ull;
    sh.hi = 0;
  }
  __syncthreads();
  {
    u64 lo = ~0ull, hi = 0;
    for_each(r.logits, r.V, [&](float l, int i) {
      if (value_bin(l) != vbin) return;
      const u64 key = composite(l, i);
      if (!member(r, l, key)) return;
      lo = key < lo ? key : lo;
      hi = key > hi ? key : hi;
    });
    if (hi != 0) {
      atomicMin(&sh.lo, lo);
      atomicMax(&sh.hi, hi);
    }
  }
  __syncthreads();
  u64 lo = sh.lo, hi = sh.hi;
  while (lo != hi) {
    const int bits = 64 - __clzll(hi - lo);
    const int shift = bits > LEVEL_BITS ? bits - LEVEL_BITS : 0;
    __syncthreads();
    for (int b = tid; b < BINS; b += TPB) {
      sh.cnt[b] = 0;
      sh.w[b] = 0;
    }
    __syncthreads();
    for_each(r.logits, r.V, [&](float l, int i) {
      const u64 key = composite(l, i);
      if (key < lo || key > hi || !member(r, l, key)) return;
      const int b = (int)((key - lo) >> shift);
      atomicAdd(&sh.cnt[b], 1u);
      if (!COUNT) atomicAdd(&sh.w[b], weight(r, l));
    });
    __syncthreads();
    const int b = pick_bin<COUNT>(need, fallback, sh);
    const u64 nlo = lo + ((u64)b << shift), nhi = nlo + ((1ull << shift) - 1);
    lo = nlo;
    hi = nhi < hi ? nhi : hi;
    if (shift == 0) break;  // the bin is one key
    // the keys that are there: mostly one, and the search is over
    if (tid == 0) {
      sh.lo = ~0ull;
      sh.hi = 0;
    }
    __syncthreads();
    u64 tlo = ~0ull, thi = 0;
    for_each(r.logits, r.V, [&](float l, int i) {
      const u64 key = composite(l, i);
      if (key < lo || key > hi || !member(r, l, key)) return;
      tlo = key < tlo ? key : tlo;
      thi = key > thi ? key : thi;
    });
    if (thi != 0) {
      atomicMin(&sh.lo, tlo);
      atomicMax(&sh.hi, thi);
    }
    __syncthreads();
    lo = sh.lo;
    hi = sh.hi;
  }
  return lo;
}

__device__ __forceinline__ float key_value(u64 key) {  // the logit of a composite key
  const uint32_t o = (uint32_t)(key >> IDX_BITS);
  return __uint_as_float((o & 0x80000000u) ? (o & 0x7fffffffu) : ~o);
}

__global__ __launch_bounds__(TPB) void sample_kernel(float* __restrict__ logits, int V, const float* __restrict__ temperature,
                                                     const int32_t* __restrict__ top_k, const float* __restrict__ top_p,
                                                     const float* __restrict__ min_p, const float* __restrict__ uniform,
                                                     int32_t* __restrict__ out_token, int32_t* __restrict__ out_candidates) {
  __shared__ Shared sh;
  const int rix = blockIdx.x, tid = threadIdx.x;
  float* row = logits + (size_t)rix * V;
  const float T = temperature[rix];
  const bool greedy = !(T > 0.f);
  const uint32_t idx_mask = (1u << IDX_BITS) - 1u;

  // The row over its temperature, written back so that the passes below read it as it counts; on the way the first
  // maximum (all that a greedy row needs; the softmax's reference point) and the smallest value.  A thread meets its
  // tokens in ascending order: a later one must be larger to take the place.
  float best = -INFINITY, least = INFINITY;
  int best_at = 0;
  for (int i0 = tid; i0 < V; i0 += 4 * TPB) {
    float v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = i0 + j * TPB < V ? row[i0 + j * TPB] : 0.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int i = i0 + j * TPB;
      if (i >= V) continue;
      float l = v[j];
      if (!greedy) {
        l = l / T;
        row[i] = l;
      }
      if (l > best || i == tid) {  // the thread's first token stands even if it is no number above -inf
        best = l;
        best_at = i;
      }
      least = fminf(least, l);
    }
  }
  u64 b = tid < V ? composite(best, best_at) : 0;
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) {
    const u64 other = __shfl_xor(b, o, kWave);
    b = other > b ? other : b;
    least = fminf(least, __shfl_xor(least, o, kWave));
  }
  __shared__ u64 wbest[TPB / kWave];
  __shared__ float wleast[TPB / kWave];
  if (tid % kWave == 0) {
    wbest[tid / kWave] = b;
    wleast[tid / kWave] = least;
  }
  __syncthreads();
  b = wbest[0];
  least = wleast[0];
  for (int w = 1; w < TPB / kWave; ++w) {
    b = wbest[w] > b ? wbest[w] : b;
    least = fminf(least, wleast[w]);
  }
  if (greedy) {  // sampler.rs:110-112
    if (tid == 0) {
      out_token[rix] = (int32_t)(idx_mask - (uint32_t)(b & idx_mask));
      out_candidates[rix] = 1;
    }
    return;
  }
  Row r;
  r.logits = row;
  r.V = V;
  r.mx = key_value(b);
  r.S = 1.f;
  r.minp_floor = 0.f;
  r.cut = 0;
  float lowest = least;
  u64 total = 0, count = 0;

  // top-k: the k-th element of the order closes the candidate set (sampler.rs:116-117)
  const int k = top_k[rix];
  if (k > 0 && k < V) {
    r.cut = select<true>(r, Target{(u64)k, 0.0, 0, false}, lowest, sh, &total, &count);
    lowest = key_value(r.cut);
  }
  const float mp = min_p[rix], tp = top_p[rix];
  u64 S = 0;  // the candidates' weight, once it is known
  if (mp > 0.f) {
    // softmax over the candidates (sampler.rs:118-126), then min-p: drop what lies below p_max * min_p, p_max being
    // the first candidate's (sampler.rs:127-130)
    u64 part = 0, none = 0;
    for_each(r.logits, r.V, [&](float l, int i) {
      if (composite(l, i) >= r.cut) part += weight(r, l);
    });
    block_totals(part, none, sh);
    S = part;
    r.S = (float)((double)S / (double)kWeightOne);
    r.minp_floor = (1.0f / r.S) * mp;
  }
  // top-p: the shortest prefix whose probability reaches top_p (sampler.rs:131-142); of the candidates' weight, which
  // without min-p is the members' and comes out of the search's own first pass
  if (tp < 1.f) {
    const u64 cut = select<false>(r, Target{0, (double)tp, S, false}, lowest, sh, &total, &count);
    r.cut = cut > r.cut ? cut : r.cut;
    lowest = key_value(r.cut);
  }
  // what is left, renormalised, and the draw (sampler.rs:143-146,155-163): the running probability must pass
  // uniform * total, the total being what the search's first pass adds up
  u64 chosen = select<false>(r, Target{0, (double)uniform[rix], 0, true}, lowest, sh, &total, &count);
  if (count <= 1) chosen = b;  // a single candidate is the first maximum
  if (tid == 0) {
    out_token[rix] = (int32_t)(idx_mask - (uint32_t)(chosen & idx_mask));
    out_candidates[rix] = (int32_t)count;
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

extern "C" int gb_sample(float* logits, int rows, int V, const float* temperature, const int32_t* top_k,
                         const float* top_p, const float* min_p, const float* uniform, int32_t* out_token,
                         int32_t* out_candidates, hipStream_t stream) {
  GB_REQUIRE(rows >= 0 && V > 0 && V <= (1 << IDX_BITS), "sample: vocabulary %d is outside 1..%d", V, 1 << IDX_BITS);
  if (rows == 0) return 0;
  hipLaunchKernelGGL(sample_kernel, dim3(rows), dim3(TPB), 0, stream, logits, V, temperature, top_k, top_p, min_p,
                     uniform, out_token, out_candidates);
  return launched("sample");
}
