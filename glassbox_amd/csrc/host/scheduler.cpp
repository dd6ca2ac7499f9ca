#include "scheduler.h"

#include <algorithm>

namespace gb {

Scheduler::Scheduler(CacheManager* cache, int token_budget, int max_seqs, int max_positions)
    : cache_(cache), token_budget_(token_budget), max_seqs_(max_seqs), max_positions_(max_positions) {}

int64_t Scheduler::submit(std::vector<int32_t> prompt, int max_tokens, const SamplerConfig& sampler,
                          std::vector<int32_t> stop) {
  // scheduler.rs:167-185
  Seq s;
  s.id = next_id_++;
  s.prompt_len = (int)prompt.size();
  s.tokens = std::move(prompt);
  s.computed = 0;
  s.max_tokens = max_tokens;
  s.sampler = sampler;
  s.rng = Rng(sampler.seed);
  s.stop = std::move(stop);
  m_prompt_ += s.prompt_len;
  int64_t id = s.id;
  waiting_.push_back(std::move(s));
  return id;
}

void Scheduler::finish_seq(Seq&& s, FinishReason reason) {
  // scheduler.rs:210-226
  if (cache_->has_seq(s.id)) cache_->remove_seq(s.id);
  if (reason != kAborted) {
    ++m_finished_;
    m_generated_ += s.generated();
  }
  finished_counts_[s.id] = {s.prompt_len, s.generated()};
  events_.push_back({s.id, 1, (int32_t)reason});
}

bool Scheduler::abort(int64_t id) {
  // scheduler.rs:200-208
  for (size_t i = 0; i < running_.size(); ++i)
    if (running_[i].id == id) {
      Seq s = std::move(running_[i]);
      running_.erase(running_.begin() + i);
      // a plan made before the abort must not be finished with stale indices
      plan_.clear();
      wants_for_.clear();
      finish_seq(std::move(s), kAborted);
      return true;
    }
  for (size_t i = 0; i < waiting_.size(); ++i)
    if (waiting_[i].id == id) {
      Seq s = std::move(waiting_[i]);
      waiting_.erase(waiting_.begin() + i);
      finish_seq(std::move(s), kAborted);
      return true;
    }
  return false;
}

bool Scheduler::preempt_last(int64_t* victim) {
  // scheduler.rs:228-236: give the pages back, recompute later, keep tokens and generator
  if (running_.empty()) return false;
  Seq s = std::move(running_.back());
  running_.pop_back();
  cache_->remove_seq(s.id);
  s.computed = 0;
  ++m_preemptions_;
  *victim = s.id;
  waiting_.push_front(std::move(s));
  return true;
}

int Scheduler::plan() {
  plan_.clear();
  wants_for_.clear();
  preempted_.clear();
  const int page = cache_->page_size();

  // admission (scheduler.rs:256-277)
  while ((int)running_.size() < max_seqs_ && !waiting_.empty()) {
    Seq& head = waiting_.front();
    int len = (int)head.tokens.size();
    // a preempted request waits until its whole context fits again
    int need = head.generated() > 0 ? (len + page - 1) / page + 1
                                    : (std::min(len, token_budget_) + page - 1) / page + 1;
    if (cache_->min_free_pages() < need && !running_.empty()) break;
    Seq s = std::move(waiting_.front());
    waiting_.pop_front();
    int reused = cache_->add_seq(s.id, s.tokens.data(), (int)s.tokens.size());
    if (reused < 0) {  // no state slot free: wait for a running request to end
      waiting_.push_front(std::move(s));
      break;
    }
    if (s.generated() == 0) m_prefix_hits_ += std::min(reused, s.prompt_len);
    s.computed = reused;
    running_.push_back(std::move(s));
  }
  if (running_.empty()) return is_idle() ? 0 : 2;

  // decoding requests first, then prompt portions, under the budget (scheduler.rs:282-298)
  std::vector<int> order(running_.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = (int)i;
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) {
    bool pa = (int)running_[a].tokens.size() - running_[a].computed > 1;
    bool pb = (int)running_[b].tokens.size() - running_[b].computed > 1;
    return pa < pb;
  });
  struct Item { int index; int n; };
  std::vector<Item> items;
  int budget = token_budget_;
  for (int i : order) {
    if (budget == 0) break;
    int n = std::min((int)running_[i].tokens.size() - running_[i].computed, budget);
    items.push_back({i, n});
    budget -= n;
  }

  // reserve pages; when they run out the newest request gives way (scheduler.rs:300-330)
  size_t k = 0;
  while (k < items.size()) {
    Item it = items[k];
    int rc = cache_->reserve(running_[it.index].id, it.n);
    if (rc == 0) {
      ++k;
      continue;
    }
    if (running_.size() == 1) {
      // alone and it still does not fit: the request is too long for the cache
      Seq s = std::move(running_.back());
      running_.pop_back();
      finish_seq(std::move(s), kLength);
      items.clear();
      break;
    }
    int64_t victim;
    preempt_last(&victim);
    preempted_.push_back(victim);
    int vi = (int)running_.size();
    for (size_t p = 0; p < items.size(); ++p)
      if (items[p].index == vi) {
        items.erase(items.begin() + p);
        if (p < k) --k;
        break;
      }
  }
  if (items.empty()) return is_idle() ? 0 : 2;

  for (auto& it : items) {
    Seq& s = running_[it.index];
    PlanEntry e;
    e.id = s.id;
    e.start = s.computed;
    e.n = it.n;
    e.wants = s.computed + it.n == (int)s.tokens.size();
    e.decode = !((int)s.tokens.size() - s.computed > 1 || s.generated() == 0);  // scheduler.rs:359-363
    e.running_index = it.index;
    plan_.push_back(e);
    if (e.wants) wants_for_.push_back(it.index);
  }
  return 1;
}

int Scheduler::planned_tokens() const {
  int n = 0;
  for (auto& e : plan_) n += e.n;
  return n;
}

void Scheduler::copy_entry_tokens(int i, int32_t* out) const {
  const PlanEntry& e = plan_[i];
  const Seq& s = running_[e.running_index];
  std::copy(s.tokens.begin() + e.start, s.tokens.begin() + e.start + e.n, out);
}

void Scheduler::row_params(int j, float* temperature, int* top_k, float* top_p, float* min_p,
                           float* repetition_penalty, float* uniform, int* skip) const {
  const Seq& s = running_[wants_for_[j]];
  *temperature = s.sampler.temperature;
  *top_k = s.sampler.top_k;
  *top_p = s.sampler.top_p;
  *min_p = s.sampler.min_p;
  *repetition_penalty = s.sampler.repetition_penalty;
  Rng peek = s.rng;
  *uniform = peek.next_f32();
  *skip = s.generated() >= s.max_tokens ? 1 : 0;  // nothing is written for it (scheduler.rs:374-378)
}

int Scheduler::row_context(int j, int32_t* out, int cap) const {
  const Seq& s = running_[wants_for_[j]];
  int n = (int)s.tokens.size();
  if (out) std::copy(s.tokens.begin(), s.tokens.begin() + std::min(n, cap), out);
  return n;
}

int Scheduler::penalty_pairs(int32_t* rows, int32_t* tokens, int32_t* counts, float* penalties, int cap) {
  int n = 0;
  for (int j = 0; j < (int)wants_for_.size(); ++j) {
    Seq& s = running_[wants_for_[j]];
    if (s.sampler.repetition_penalty == 1.0f) continue;
    for (; s.counted < s.tokens.size(); ++s.counted) ++s.occurrences[s.tokens[s.counted]];
    for (const auto& kv : s.occurrences) {
      if (n < cap) {
        rows[n] = j;
        tokens[n] = kv.first;
        counts[n] = kv.second;
        penalties[n] = s.sampler.repetition_penalty;
      }
      ++n;
    }
  }
  return n;
}

void Scheduler::finish(const int32_t* sampled, const int32_t* n_candidates, int n_rows) {
  if (plan_.empty()) return;
  // commit what the step wrote (scheduler.rs:356-368)
  int batch_tokens = 0;
  for (auto& e : plan_) {
    Seq& s = running_[e.running_index];
    cache_->commit(s.id, s.tokens.data() + e.start, e.n);
    s.computed += e.n;
    batch_tokens += e.n;
  }
  // sample results, stop and length checks (scheduler.rs:370-404)
  std::vector<std::pair<int, FinishReason>> done;
  for (int j = 0; j < (int)wants_for_.size() && j < n_rows; ++j) {
    int i = wants_for_[j];
    Seq& s = running_[i];
    if (s.generated() >= s.max_tokens) {
      done.push_back({i, kLength});
      continue;
    }
    int32_t t = sampled[j];
    // the uniform number was drawn from a copy; it counts only if a draw took place
    // (crates/glassbox-core/src/sampler.rs:152-155)
    if (s.sampler.temperature > 0.f && n_candidates[j] > 1) s.rng.next_f32();
    bool stop = std::find(s.stop.begin(), s.stop.end(), t) != s.stop.end();
    if (!stop) {
      s.tokens.push_back(t);
      events_.push_back({s.id, 0, t});
    }
    if (stop) done.push_back({i, kStop});
    else if (s.generated() >= s.max_tokens || (int)s.tokens.size() >= max_positions_) done.push_back({i, kLength});
  }
  std::sort(done.begin(), done.end(), [](auto& a, auto& b) { return a.first > b.first; });
  for (auto& d : done) {
    Seq s = std::move(running_[d.first]);
    running_.erase(running_.begin() + d.first);
    finish_seq(std::move(s), d.second);
  }
  ++m_steps_;
  m_batch_tokens_ += batch_tokens;
  plan_.clear();
  wants_for_.clear();
}

int Scheduler::take_events(int64_t* ids, int32_t* kinds, int32_t* values, int cap) {
  int n = (int)events_.size();
  int give = std::min(n, cap);
  for (int i = 0; i < give; ++i) {
    ids[i] = events_[i].id;
    kinds[i] = events_[i].kind;
    values[i] = events_[i].value;
  }
  events_.erase(events_.begin(), events_.begin() + give);
  return n;
}

bool Scheduler::request_counts(int64_t id, int* prompt_tokens, int* completion_tokens) const {
  auto it = finished_counts_.find(id);
  if (it == finished_counts_.end()) return false;
  *prompt_tokens = it->second.prompt;
  *completion_tokens = it->second.completion;
  return true;
}

void Scheduler::metrics(int64_t* out7) const {
  out7[0] = m_finished_;
  out7[1] = m_prompt_;
  out7[2] = m_generated_;
  out7[3] = m_prefix_hits_;
  out7[4] = m_preemptions_;
  out7[5] = m_steps_;
  out7[6] = m_batch_tokens_;
}

int Scheduler::last_preempted(int64_t* out, int cap) const {
  int n = (int)preempted_.size();
  for (int i = 0; i < n && i < cap; ++i) out[i] = preempted_[i];
  return n;
}

}  // namespace gb
