// Continuous batching above the step function: admits requests, cuts prompts into
// portions under a token budget, lets decoding requests go first, preempts the most
// recently admitted request when pages run out, finishes and frees.
//
// The decisions follow the reference's Scheduler (crates/glassbox-server/src/scheduler.rs).
// One reference step() is split in two here because the model runs on the device in
// between: plan() decides the batch and reserves its pages, the engine runs the batch
// and samples, finish() commits, appends the sampled tokens and retires requests.
#pragma once
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"
#include "sampler.h"

namespace gb {

enum FinishReason : int { kStop = 0, kLength = 1, kAborted = 2 };

struct PlanEntry {
  int64_t id;
  int start;     // position of the first token of this portion
  int n;         // tokens in this portion
  bool wants;    // the portion ends the known tokens: logits of its last token are needed
  bool decode;   // a single generated token (for step records)
  int running_index;
};

class Scheduler {
 public:
  Scheduler(CacheManager* cache, int token_budget, int max_seqs, int max_positions);

  int64_t submit(std::vector<int32_t> prompt, int max_tokens, const SamplerConfig& sampler,
                 std::vector<int32_t> stop);
  bool abort(int64_t id);
  bool is_idle() const { return waiting_.empty() && running_.empty(); }
  int waiting() const { return (int)waiting_.size(); }
  int running() const { return (int)running_.size(); }

  int plan();
  const std::vector<PlanEntry>& planned() const { return plan_; }
  int planned_tokens() const;
  void copy_entry_tokens(int i, int32_t* out) const;
  void row_params(int j, float* temperature, int* top_k, float* top_p, float* min_p, float* repetition_penalty,
                  float* uniform, int* skip) const;
  int row_context(int j, int32_t* out, int cap) const;
  void finish(const int32_t* sampled, const int32_t* n_candidates, int n_rows);

  // The repetition penalty of the wanted rows as (row, token, occurrences, penalty), one for every distinct token of
  // a row whose request has a penalty other than 1.  Returns how many there are; fills at most `cap`.
  int penalty_pairs(int32_t* rows, int32_t* tokens, int32_t* counts, float* penalties, int cap);
  int take_events(int64_t* ids, int32_t* kinds, int32_t* values, int cap);
  bool request_counts(int64_t id, int* prompt_tokens, int* completion_tokens) const;
  void metrics(int64_t* out7) const;
  int last_preempted(int64_t* out, int cap) const;

 private:
  struct Seq {
    int64_t id;
    std::vector<int32_t> tokens;  // prompt then generated
    int prompt_len;
    int computed;                 // tokens whose keys and values are in the cache
    int max_tokens;
    SamplerConfig sampler;
    Rng rng;
    std::vector<int32_t> stop;
    // how often each token occurs among the first `counted` tokens: kept for requests with a repetition penalty,
    // brought up to date when their penalty is asked for, so that a step costs what it adds and not the context
    std::unordered_map<int32_t, int32_t> occurrences;
    size_t counted = 0;
    int generated() const { return (int)tokens.size() - prompt_len; }
  };
  struct Event { int64_t id; int32_t kind; int32_t value; };
  struct Counts { int prompt; int completion; };

  void finish_seq(Seq&& s, FinishReason reason);
  bool preempt_last(int64_t* victim);

  CacheManager* cache_;
  int token_budget_, max_seqs_, max_positions_;
  std::deque<Seq> waiting_;
  std::vector<Seq> running_;
  int64_t next_id_ = 1;
  std::vector<PlanEntry> plan_;
  std::vector<int> wants_for_;     // running index of each wanted row
  std::vector<Event> events_;
  std::vector<int64_t> preempted_;
  std::unordered_map<int64_t, Counts> finished_counts_;
  int64_t m_finished_ = 0, m_prompt_ = 0, m_generated_ = 0, m_prefix_hits_ = 0, m_preemptions_ = 0,
          m_steps_ = 0, m_batch_tokens_ = 0;
};

}  // namespace gb
