// Host-side sampler: the scalar twin of the device sampling kernels and the owner of
// each request's random number generator.  Formulas and their order follow the
// reference (crates/glassbox-core/src/sampler.rs:3-164).
#pragma once
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <numeric>
#include <utility>
#include <vector>

namespace gb {

struct SamplerConfig {
  float temperature = 0.f;         // 0 (or less) = greedy            sampler.rs:5-6
  int top_k = 0;                   // 0 disables                       sampler.rs:7-8
  float top_p = 1.f;               // 1 disables                       sampler.rs:9-10
  float min_p = 0.f;               // 0 disables                       sampler.rs:11-12
  float repetition_penalty = 1.f;  // 1 disables                       sampler.rs:13-14
  uint64_t seed = 0;
};

// xorshift64* (sampler.rs:33-47)
struct Rng {
  uint64_t state = 1;
  Rng() = default;
  explicit Rng(uint64_t seed) : state(seed * 0x9e3779b97f4a7c15ull | 1ull) {}
  float next_f32() {
    state ^= state >> 12;
    state ^= state << 25;
    state ^= state >> 27;
    uint64_t x = state * 0x2545f4914f6cdd1dull;
    return (float)(x >> 40) / (float)(1ull << 24);
  }
};

// first maximum wins (sampler.rs:49-57)
inline int argmax(const float* x, int n) {
  int best = 0;
  for (int i = 1; i < n; ++i)
    if (x[i] > x[best]) best = i;
  return best;
}

// The distribution after every filter, most likely first (sampler.rs:97-148).  Equal values
// are ordered by token id, which the reference leaves to an unstable selection.
inline std::vector<std::pair<int, float>> distribution(const SamplerConfig& c, const float* logits, int vocab,
                                                       const int32_t* context, int n_context) {
  std::vector<float> l(logits, logits + vocab);
  if (c.repetition_penalty != 1.f) {
    for (int i = 0; i < n_context; ++i) {
      float& v = l[context[i]];
      v = v > 0.f ? v / c.repetition_penalty : v * c.repetition_penalty;
    }
  }
  if (c.temperature <= 0.f) return {{argmax(l.data(), vocab), 1.f}};
  for (float& v : l) v /= c.temperature;
  int k = c.top_k == 0 ? vocab : std::min(c.top_k, vocab);
  std::vector<int> idx(vocab);
  std::iota(idx.begin(), idx.end(), 0);
  std::stable_sort(idx.begin(), idx.end(), [&](int a, int b) { return l[a] > l[b]; });
  idx.resize(k);
  std::vector<std::pair<int, float>> cand;
  cand.reserve(k);
  float max = l[idx[0]], sum = 0.f;
  for (int i : idx) {
    float e = std::exp(l[i] - max);
    sum += e;
    cand.emplace_back(i, e);
  }
  for (auto& p : cand) p.second /= sum;
  if (c.min_p > 0.f) {
    float floor = cand[0].second * c.min_p;
    cand.erase(std::remove_if(cand.begin(), cand.end(), [&](auto& p) { return p.second < floor; }), cand.end());
  }
  if (c.top_p < 1.f) {
    float acc = 0.f;
    size_t keep = cand.size();
    for (size_t i = 0; i < cand.size(); ++i) {
      acc += cand[i].second;
      if (acc >= c.top_p) { keep = i + 1; break; }
    }
    cand.resize(keep);
  }
  float total = 0.f;
  for (auto& p : cand) total += p.second;
  for (auto& p : cand) p.second /= total;
  return cand;
}

// sampler.rs:150-164: no draw when one candidate is left
inline int sample(const SamplerConfig& c, Rng& rng, const float* logits, int vocab, const int32_t* context,
                  int n_context) {
  auto dist = distribution(c, logits, vocab, context, n_context);
  if (dist.size() == 1) return dist[0].first;
  float r = rng.next_f32(), acc = 0.f;
  for (auto& p : dist) {
    acc += p.second;
    if (r < acc) return p.first;
  }
  return dist.back().first;
}

}  // namespace gb
