// C interface of the host runtime (cache manager, scheduler, sampler), loaded
// from Python through ctypes.  Every object is an opaque handle.
#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "cache_manager.h"
#include "sampler.h"
#include "scheduler.h"

using gb::CacheManager;

extern "C" {

// ---- cache manager -------------------------------------------------------
void* gbh_cache_create(int page_size, int n_groups, const int* kinds, const int* windows,
                       const int* num_pages, int num_state_slots, int share_prefixes) {
  std::vector<gb::GroupSpec> groups(n_groups);
  for (int i = 0; i < n_groups; ++i) {
    groups[i].kind = kinds[i];
    groups[i].window = windows[i];
    groups[i].num_pages = num_pages[i];
  }
  return new CacheManager(page_size, groups, num_state_slots, share_prefixes != 0);
}
void gbh_cache_destroy(void* h) { delete (CacheManager*)h; }
int gbh_cache_add_seq(void* h, int64_t id, const int32_t* prompt, int n) { return ((CacheManager*)h)->add_seq(id, prompt, n); }
int gbh_cache_reserve(void* h, int64_t id, int n) { return ((CacheManager*)h)->reserve(id, n); }
int gbh_cache_commit(void* h, int64_t id, const int32_t* tokens, int n) { return ((CacheManager*)h)->commit(id, tokens, n); }
int gbh_cache_truncate(void* h, int64_t id, int len) { return ((CacheManager*)h)->truncate(id, len); }
int gbh_cache_fork(void* h, int64_t parent, int64_t child) { return ((CacheManager*)h)->fork(parent, child); }
int gbh_cache_remove_seq(void* h, int64_t id) { return ((CacheManager*)h)->remove_seq(id); }
int gbh_cache_has_seq(void* h, int64_t id) { return ((CacheManager*)h)->has_seq(id) ? 1 : 0; }
int gbh_cache_seq_len(void* h, int64_t id) { return ((CacheManager*)h)->seq_len(id); }
int gbh_cache_state_slot(void* h, int64_t id) { return ((CacheManager*)h)->state_slot(id); }
int gbh_cache_free_pages(void* h, int g) { return ((CacheManager*)h)->free_pages(g); }
int gbh_cache_min_free_pages(void* h) { return ((CacheManager*)h)->min_free_pages(); }
int gbh_cache_num_pages(void* h, int g) { return ((CacheManager*)h)->num_pages(g); }
int gbh_cache_ref_count(void* h, int g, int page) { return ((CacheManager*)h)->ref_count(g, page); }
int gbh_cache_free_state_slots(void* h) { return ((CacheManager*)h)->free_state_slots(); }
int gbh_cache_num_seqs(void* h) { return ((CacheManager*)h)->num_seqs(); }
int gbh_cache_share_prefixes(void* h) { return ((CacheManager*)h)->share_prefixes() ? 1 : 0; }
int gbh_cache_pages_needed(void* h, int64_t id, int n) { return ((CacheManager*)h)->pages_needed(id, n); }
// Copies the request's table of `group` into out (at most cap entries); returns its length or -1.
int gbh_cache_table(void* h, int64_t id, int group, int32_t* out, int cap) {
  auto* t = ((CacheManager*)h)->table(id, group);
  if (!t) return -1;
  int n = (int)t->size();
  if (out) std::memcpy(out, t->data(), sizeof(int32_t) * (size_t)(n < cap ? n : cap));
  return n;
}
// What a step of one token per request needs, written straight into the caller's (pinned) arrays: per request
// its length (the new token's position) and state slot, and per group the cache row of the new token and the
// block table, padded with -1 to `stride` entries.  rows and tables are laid out [group][request] and
// [group][request][stride], with `group_gap` entries from one group's array to the next.  Returns 0; -1 for an
// unknown request; -2 if a table is longer than stride; -3 if the page of the new position is not reserved.
// ahead (may be null): tokens of request i that an earlier step has brought and that are not committed yet; the
// new token's position lies that many beyond the request's length (a step launched before the one before it
// has been accounted for).
int gbh_cache_decode_rows(void* h, const int64_t* ids, int n, int stride, int32_t* pos, int32_t* state_slot,
                          int32_t* rows, int rows_gap, int32_t* tables, int tables_gap, const int32_t* ahead) {
  auto* cm = (CacheManager*)h;
  const int page = cm->page_size(), groups = cm->num_groups();
  for (int i = 0; i < n; ++i) {
    int len = cm->seq_len(ids[i]);
    if (len < 0) return -1;
    if (ahead) len += ahead[i];
    pos[i] = len;
    state_slot[i] = cm->state_slot(ids[i]);
    for (int g = 0; g < groups; ++g) {
      const std::vector<int32_t>& t = *cm->table(ids[i], g);
      if ((int)t.size() > stride) return -2;
      int32_t* out = tables + (size_t)g * tables_gap + (size_t)i * stride;
      std::memcpy(out, t.data(), sizeof(int32_t) * t.size());
      for (int j = (int)t.size(); j < stride; ++j) out[j] = -1;
      int lp = len / page;
      if (lp >= (int)t.size() || t[lp] < 0) return -3;
      rows[(size_t)g * rows_gap + i] = t[lp] * page + len % page;
    }
  }
  return 0;
}
// The same for a step of any mix: request i brings counts[i] tokens at positions len .. len + counts[i] - 1.
// Per token (requests in the order given, their tokens in order): position, index of its request, and per group
// the cache row ([group][token], rows_gap entries between groups).  Per request: first token's index, first
// position, state slot, and per group the block table padded with -1 to `stride` entries.  Returns 0; -1 for an
// unknown request; -3 if a position is not reserved; the stride that is needed if `stride` is too small.
int gbh_cache_step_rows(void* h, const int64_t* ids, const int32_t* counts, int n, int stride, int32_t* positions,
                        int32_t* tok_seq, int32_t* q_start, int32_t* pos0, int32_t* state_slot, int32_t* rows,
                        int rows_gap, int32_t* tables, int tables_gap) {
  auto* cm = (CacheManager*)h;
  const int page = cm->page_size(), groups = cm->num_groups();
  int need = 0;
  for (int i = 0; i < n; ++i) {
    if (cm->seq_len(ids[i]) < 0) return -1;
    for (int g = 0; g < groups; ++g) need = std::max(need, (int)cm->table(ids[i], g)->size());
  }
  if (need > stride) return need;
  int at = 0;
  for (int i = 0; i < n; ++i) {
    const int len = cm->seq_len(ids[i]);
    q_start[i] = at;
    pos0[i] = len;
    state_slot[i] = cm->state_slot(ids[i]);
    for (int j = 0; j < counts[i]; ++j) {
      positions[at + j] = len + j;
      tok_seq[at + j] = i;
    }
    for (int g = 0; g < groups; ++g) {
      const std::vector<int32_t>& t = *cm->table(ids[i], g);
      int32_t* out = tables + (size_t)g * tables_gap + (size_t)i * stride;
      std::memcpy(out, t.data(), sizeof(int32_t) * t.size());
      for (int j = (int)t.size(); j < stride; ++j) out[j] = -1;
      for (int j = 0; j < counts[i]; ++j) {
        const int p = len + j, lp = p / page;
        if (lp >= (int)t.size() || t[lp] < 0) return -3;
        rows[(size_t)g * rows_gap + at + j] = t[lp] * page + p % page;
      }
    }
    at += counts[i];
  }
  return 0;
}
// Pending device copies as triples (group, src, dst); returns how many there were.
int gbh_cache_take_copies(void* h, int32_t* out, int cap_triples) {
  auto ops = ((CacheManager*)h)->take_copies();
  int n = (int)ops.size();
  for (int i = 0; i < n && i < cap_triples; ++i) {
    out[3 * i] = ops[i].group;
    out[3 * i + 1] = ops[i].src;
    out[3 * i + 2] = ops[i].dst;
  }
  return n;
}
int gbh_cache_check(void* h, char* why, int cap) {
  std::string msg;
  bool ok = ((CacheManager*)h)->check_invariants(&msg);
  if (why && cap > 0) {
    std::strncpy(why, msg.c_str(), (size_t)cap - 1);
    why[cap - 1] = 0;
  }
  return ok ? 1 : 0;
}
uint64_t gbh_chain_hash(uint64_t prev, const int32_t* tokens, int n) { return gb::chain_hash(prev, tokens, n); }

// ---- sampler -------------------------------------------------------------
uint64_t gbh_rng_new(uint64_t seed) { return gb::Rng(seed).state; }
float gbh_rng_next(uint64_t* state) {
  gb::Rng r;
  r.state = *state;
  float v = r.next_f32();
  *state = r.state;
  return v;
}
// Host sampler over one row of logits: returns the token; advances *rng_state only when a
// draw was needed.  It is the scalar twin of the device sampling kernels and serves tests.
int gbh_sample(const float* logits, int vocab, const int32_t* context, int n_context, float temperature,
               int top_k, float top_p, float min_p, float repetition_penalty, uint64_t* rng_state) {
  gb::SamplerConfig c;
  c.temperature = temperature;
  c.top_k = top_k;
  c.top_p = top_p;
  c.min_p = min_p;
  c.repetition_penalty = repetition_penalty;
  gb::Rng r;
  r.state = *rng_state;
  int t = gb::sample(c, r, logits, vocab, context, n_context);
  *rng_state = r.state;
  return t;
}

// ---- scheduler -----------------------------------------------------------
void* gbh_sched_create(void* cache, int token_budget, int max_seqs, int max_positions) {
  return new gb::Scheduler((CacheManager*)cache, token_budget, max_seqs, max_positions);
}
void gbh_sched_destroy(void* h) { delete (gb::Scheduler*)h; }
int64_t gbh_sched_submit(void* h, const int32_t* prompt, int n, int max_tokens, float temperature, int top_k,
                         float top_p, float min_p, float repetition_penalty, uint64_t seed,
                         const int32_t* stop, int n_stop) {
  gb::SamplerConfig c;
  c.temperature = temperature;
  c.top_k = top_k;
  c.top_p = top_p;
  c.min_p = min_p;
  c.repetition_penalty = repetition_penalty;
  c.seed = seed;
  return ((gb::Scheduler*)h)->submit(std::vector<int32_t>(prompt, prompt + n), max_tokens, c,
                                     std::vector<int32_t>(stop, stop + n_stop));
}
int gbh_sched_abort(void* h, int64_t id) { return ((gb::Scheduler*)h)->abort(id) ? 1 : 0; }
int gbh_sched_is_idle(void* h) { return ((gb::Scheduler*)h)->is_idle() ? 1 : 0; }
int gbh_sched_waiting(void* h) { return ((gb::Scheduler*)h)->waiting(); }
int gbh_sched_running(void* h) { return ((gb::Scheduler*)h)->running(); }
// Plans one step.  Returns 0 = nothing to run and idle, 1 = a batch is planned, 2 = nothing
// planned this time but work remains.
int gbh_sched_plan(void* h) { return ((gb::Scheduler*)h)->plan(); }
int gbh_sched_plan_size(void* h) { return (int)((gb::Scheduler*)h)->planned().size(); }
int gbh_sched_plan_tokens(void* h) { return ((gb::Scheduler*)h)->planned_tokens(); }
// Entry i of the plan: id, start position, token count, wants logits (0/1), decode (0/1).
void gbh_sched_plan_entry(void* h, int i, int64_t* id, int* start, int* n, int* wants, int* is_decode) {
  auto& e = ((gb::Scheduler*)h)->planned()[i];
  *id = e.id;
  *start = e.start;
  *n = e.n;
  *wants = e.wants ? 1 : 0;
  *is_decode = e.decode ? 1 : 0;
}
// Copies the tokens of plan entry i (n of them) into out.
void gbh_sched_plan_entry_tokens(void* h, int i, int32_t* out) { ((gb::Scheduler*)h)->copy_entry_tokens(i, out); }
// The whole plan in one call: per entry id, start, count, wants, decode (arrays of plan_size entries) and all
// entries' tokens one after the other (plan_tokens of them).
void gbh_sched_plan_all(void* h, int64_t* ids, int32_t* starts, int32_t* counts, int32_t* wants, int32_t* decodes,
                        int32_t* tokens) {
  auto* s = (gb::Scheduler*)h;
  const auto& plan = s->planned();
  int at = 0;
  for (size_t i = 0; i < plan.size(); ++i) {
    ids[i] = plan[i].id;
    starts[i] = plan[i].start;
    counts[i] = plan[i].n;
    wants[i] = plan[i].wants ? 1 : 0;
    decodes[i] = plan[i].decode ? 1 : 0;
    s->copy_entry_tokens((int)i, tokens + at);
    at += plan[i].n;
  }
}
// Sampling parameters of the wanted rows 0 .. n-1 in one call (arrays of n entries; see gbh_sched_row_params).
void gbh_sched_rows_params(void* h, int n, float* temperature, int32_t* top_k, float* top_p, float* min_p,
                           float* repetition_penalty, float* uniform, int32_t* skip) {
  for (int j = 0; j < n; ++j) {
    int k = 0, sk = 0;
    ((gb::Scheduler*)h)->row_params(j, temperature + j, &k, top_p + j, min_p + j, repetition_penalty + j, uniform + j, &sk);
    top_k[j] = k;
    skip[j] = sk;
  }
}
// The longest of the requests' lengths (-1 for an unknown request).
int gbh_cache_max_len(void* h, const int64_t* ids, int n) {
  int longest = 0;
  for (int i = 0; i < n; ++i) {
    const int len = ((CacheManager*)h)->seq_len(ids[i]);
    if (len < 0) return -1;
    longest = std::max(longest, len);
  }
  return longest;
}
// The longest block table among the requests, in pages, over all groups (-1 for an unknown request).  A request
// may hold more pages than its length needs: a reservation that was never committed keeps them.
int gbh_cache_max_pages(void* h, const int64_t* ids, int n) {
  auto* cm = (CacheManager*)h;
  int longest = 0;
  for (int i = 0; i < n; ++i) {
    if (cm->seq_len(ids[i]) < 0) return -1;
    for (int g = 0; g < cm->num_groups(); ++g) longest = std::max(longest, (int)cm->table(ids[i], g)->size());
  }
  return longest;
}
// Sampling parameters of the j-th wanted row, with a uniform number drawn ahead from a copy of
// the request's generator (the draw is kept only if the device reports more than one candidate).
void gbh_sched_row_params(void* h, int j, float* temperature, int* top_k, float* top_p, float* min_p,
                          float* repetition_penalty, float* uniform, int* skip) {
  ((gb::Scheduler*)h)->row_params(j, temperature, top_k, top_p, min_p, repetition_penalty, uniform, skip);
}
// Tokens (prompt and generated) of the request behind wanted row j: the penalty's context.
int gbh_sched_row_context(void* h, int j, int32_t* out, int cap) { return ((gb::Scheduler*)h)->row_context(j, out, cap); }
// The repetition penalty's work for the wanted rows: (row, token, occurrences, penalty) for every distinct token of
// a row with a penalty; returns their number (ask with cap 0, then fill).
int gbh_sched_penalty_pairs(void* h, int32_t* rows, int32_t* tokens, int32_t* counts, float* penalties, int cap) {
  return ((gb::Scheduler*)h)->penalty_pairs(rows, tokens, counts, penalties, cap);
}
// Finishes the planned step: commits, appends sampled tokens (one per wanted row, with how many
// candidates the draw had), finishes requests.
void gbh_sched_finish(void* h, const int32_t* sampled, const int32_t* n_candidates, int n_rows) {
  ((gb::Scheduler*)h)->finish(sampled, n_candidates, n_rows);
}
// Events since the last call, as (id, kind, value): kind 0 = token, 1 = done with reason in value
// (0 stop, 1 length, 2 aborted).  Returns how many there were.
int gbh_sched_take_events(void* h, int64_t* ids, int32_t* kinds, int32_t* values, int cap) {
  return ((gb::Scheduler*)h)->take_events(ids, kinds, values, cap);
}
int gbh_sched_request_counts(void* h, int64_t id, int* prompt_tokens, int* completion_tokens) {
  return ((gb::Scheduler*)h)->request_counts(id, prompt_tokens, completion_tokens) ? 1 : 0;
}
// requests_finished, prompt_tokens, generated_tokens, prefix_hit_tokens, preemptions, steps, batch_tokens
void gbh_sched_metrics(void* h, int64_t* out7) { ((gb::Scheduler*)h)->metrics(out7); }
// Preempted and finished ids of the last plan()/finish() pair, for step records.
int gbh_sched_last_preempted(void* h, int64_t* out, int cap) { return ((gb::Scheduler*)h)->last_preempted(out, cap); }

}  // extern "C"
