#include "cache_manager.h"

#include <algorithm>
#include <sstream>

namespace gb {

uint64_t chain_hash(uint64_t prev, const int32_t* tokens, int n) {
  // FNV-1a over the previous hash and the page's tokens as little-endian bytes (kv.rs:45-55)
  uint64_t h = prev ^ 0xcbf29ce484222325ull;
  for (int i = 0; i < n; ++i) {
    uint32_t t = (uint32_t)tokens[i];
    for (int b = 0; b < 4; ++b) {
      h ^= (uint64_t)((t >> (8 * b)) & 0xff);
      h *= 0x100000001b3ull;
    }
  }
  return h;
}

CacheManager::CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots,
                           bool share_prefixes)
    : page_size_(page_size), num_state_slots_(num_state_slots), share_(share_prefixes) {
  for (auto& spec : groups) {
    Group g;
    g.spec = spec;
    g.refs.assign(spec.num_pages, 0);
    g.free.reserve(spec.num_pages);
    for (int p = spec.num_pages - 1; p >= 0; --p) g.free.push_back(p);  // kv.rs:67
    g.page_hash.assign(spec.num_pages, 0);
    g.has_hash.assign(spec.num_pages, 0);
    // a page a window has passed is gone, so its prefix cannot be offered to others
    if (spec.kind != kFull) share_ = false;
    groups_.push_back(std::move(g));
  }
  for (int s = num_state_slots - 1; s >= 0; --s) free_slots_.push_back(s);
}

int CacheManager::alloc(Group& g) {
  int32_t page;
  if (!g.free.empty()) {
    page = g.free.back();
    g.free.pop_back();
  } else if (!g.cached.empty()) {
    // evict the oldest idle page that was kept for its prefix (kv.rs:99-105)
    page = g.cached.front();
    g.cached.erase(g.cached.begin());
    if (g.has_hash[page]) {
      g.by_hash.erase(g.page_hash[page]);
      g.has_hash[page] = 0;
    }
  } else {
    return -1;
  }
  g.refs[page] = 1;
  return page;
}

void CacheManager::release(Group& g, int32_t page) {
  if (--g.refs[page] == 0) {
    if (g.has_hash[page]) g.cached.push_back(page);
    else g.free.push_back(page);
    // a copy into this page that the engine has not made yet is void: the page may be handed out again, as
    // another copy's destination too, and two copies into one page would land in an undefined order
    drop_copies_into((int)(&g - groups_.data()), page);
  }
}

void CacheManager::drop_copies_into(int group, int32_t dst) {
  copies_.erase(std::remove_if(copies_.begin(), copies_.end(),
                               [&](const CopyOp& c) { return c.group == group && c.dst == dst; }),
                copies_.end());
}

void CacheManager::retain(Group& g, int32_t page) {
  if (g.refs[page] == 0) g.cached.erase(std::remove(g.cached.begin(), g.cached.end(), page), g.cached.end());
  ++g.refs[page];
}

int CacheManager::add_seq(int64_t id, const int32_t* prompt, int n) {
  if (seqs_.count(id)) return -1;
  Seq s;
  if (num_state_slots_ > 0) {
    if (free_slots_.empty()) return -2;
    s.state_slot = free_slots_.back();
    free_slots_.pop_back();
  }
  s.tables.resize(groups_.size());
  s.tokens.assign(prompt, prompt + n);
  uint64_t h = 0;
  int pages = 0;
  for (int c = 0; share_ && (c + 1) * page_size_ <= n; ++c) {
    if ((pages + 1) * page_size_ >= n) break;  // the last token always runs (kv.rs:143)
    h = chain_hash(h, prompt + c * page_size_, page_size_);
    bool everywhere = true;
    for (auto& g : groups_)
      if (!g.by_hash.count(h)) { everywhere = false; break; }
    if (!everywhere) break;
    for (size_t gi = 0; gi < groups_.size(); ++gi) {
      int32_t page = groups_[gi].by_hash[h];
      retain(groups_[gi], page);
      s.tables[gi].push_back(page);
    }
    ++pages;
  }
  s.len = pages * page_size_;
  int reused = s.len;
  seqs_.emplace(id, std::move(s));
  return reused;
}

int CacheManager::need_in_group(const Seq& s, int gi, int n) const {
  const Group& g = groups_[gi];
  int need = (s.len + n + page_size_ - 1) / page_size_ - (int)s.tables[gi].size();
  if (need < 0) need = 0;
  if (s.len % page_size_ != 0) {
    int32_t last = s.tables[gi][s.len / page_size_];
    if (last >= 0 && g.refs[last] > 1) ++need;  // the copy-on-write page
  }
  return need;
}

int CacheManager::pages_needed(int64_t id, int n) const {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) return -1;
  int most = 0;
  for (size_t gi = 0; gi < groups_.size(); ++gi) most = std::max(most, need_in_group(it->second, (int)gi, n));
  return most;
}

int CacheManager::reserve(int64_t id, int n) {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) return -1;
  Seq& s = it->second;
  // all or nothing, over every group (kv.rs:165-169)
  for (size_t gi = 0; gi < groups_.size(); ++gi)
    if (need_in_group(s, (int)gi, n) > free_pages((int)gi)) return 1;
  for (size_t gi = 0; gi < groups_.size(); ++gi) {
    Group& g = groups_[gi];
    auto& table = s.tables[gi];
    if (s.len % page_size_ != 0) {
      int idx = s.len / page_size_;
      int32_t last = table[idx];
      if (last >= 0 && g.refs[last] > 1) {  // copy-on-write (kv.rs:171-181)
        int fresh = alloc(g);
        copies_.push_back({(int)gi, last, fresh});
        release(g, last);
        table[idx] = fresh;
      }
    }
    int want = (s.len + n + page_size_ - 1) / page_size_;
    while ((int)table.size() < want) table.push_back(alloc(g));
  }
  return 0;
}

int CacheManager::commit(int64_t id, const int32_t* tokens, int n) {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) return -1;
  Seq& s = it->second;
  int start = s.len;
  s.len += n;
  if ((int)s.tokens.size() < s.len) {  // kv.rs:209-212
    s.tokens.resize(start);
    s.tokens.insert(s.tokens.end(), tokens, tokens + n);
  }
  if (share_) {
    int first_full = start / page_size_, last_full = s.len / page_size_;
    for (int bi = first_full; bi < last_full; ++bi) {
      uint64_t h = 0;
      bool hashed = false;
      for (size_t gi = 0; gi < groups_.size(); ++gi) {
        Group& g = groups_[gi];
        int32_t page = s.tables[gi][bi];
        if (page < 0 || g.has_hash[page]) continue;
        if (!hashed) {
          for (int c = 0; c <= bi; ++c) h = chain_hash(h, s.tokens.data() + c * page_size_, page_size_);
          hashed = true;
        }
        if (!g.by_hash.count(h)) {  // first page with this prefix keeps the registration (kv.rs:228-231)
          g.by_hash[h] = page;
          g.page_hash[page] = h;
          g.has_hash[page] = 1;
        }
      }
    }
  }
  // pages that every later query's window has passed go back to their pool
  for (size_t gi = 0; gi < groups_.size(); ++gi) {
    Group& g = groups_[gi];
    if (g.spec.kind != kWindow) continue;
    int first_needed = s.len - g.spec.window + 1;  // oldest key the next query reads
    if (first_needed <= 0) continue;
    int dead = first_needed / page_size_;          // pages [0, dead) lie wholly before it
    auto& table = s.tables[gi];
    for (int j = 0; j < dead && j < (int)table.size(); ++j) {
      if (table[j] >= 0) {
        release(g, table[j]);
        table[j] = -1;
      }
    }
  }
  return 0;
}

int CacheManager::truncate(int64_t id, int len) {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) return -1;
  Seq& s = it->second;
  if (len > s.len || len < 0) return -2;
  for (size_t gi = 0; gi < groups_.size(); ++gi) {
    const Group& g = groups_[gi];
    if (g.spec.kind != kWindow) continue;
    int first_needed = std::max(0, len - g.spec.window + 1);
    for (int j = first_needed / page_size_; j < (len + page_size_ - 1) / page_size_; ++j)
      if (s.tables[gi][j] < 0) return -3;  // the window would reach into pages already given back
  }
  s.len = len;
  if ((int)s.tokens.size() > len) s.tokens.resize(len);
  int keep = (len + page_size_ - 1) / page_size_;
  for (size_t gi = 0; gi < groups_.size(); ++gi) {
    Group& g = groups_[gi];
    auto& table = s.tables[gi];
    std::vector<int32_t> dropped(table.begin() + std::min<size_t>(keep, table.size()), table.end());
    table.resize(std::min<size_t>(keep, table.size()));
    if (len % page_size_ != 0) {
      // the last kept page will be rewritten: its prefix hash no longer describes it (kv.rs:244-253)
      int32_t page = table[len / page_size_];
      if (page >= 0 && g.refs[page] == 1 && g.has_hash[page]) {
        g.by_hash.erase(g.page_hash[page]);
        g.has_hash[page] = 0;
      }
    }
    for (int32_t page : dropped)
      if (page >= 0) release(g, page);
  }
  return 0;
}

int CacheManager::fork(int64_t parent, int64_t child) {
  auto it = seqs_.find(parent);
  if (it == seqs_.end()) return -1;
  if (seqs_.count(child)) return -2;
  Seq s = it->second;
  if (num_state_slots_ > 0) {
    if (free_slots_.empty()) return -3;
    s.state_slot = free_slots_.back();
    free_slots_.pop_back();
    copies_.push_back({-1, it->second.state_slot, s.state_slot});
  }
  for (size_t gi = 0; gi < groups_.size(); ++gi)
    for (int32_t page : s.tables[gi])
      if (page >= 0) retain(groups_[gi], page);
  seqs_.emplace(child, std::move(s));
  return 0;
}

int CacheManager::remove_seq(int64_t id) {
  auto it = seqs_.find(id);
  if (it == seqs_.end()) return -1;
  Seq& s = it->second;
  for (size_t gi = 0; gi < groups_.size(); ++gi)
    for (int32_t page : s.tables[gi])
      if (page >= 0) release(groups_[gi], page);
  if (s.state_slot >= 0) {
    free_slots_.push_back(s.state_slot);
    drop_copies_into(-1, s.state_slot);
  }
  seqs_.erase(it);
  return 0;
}

int CacheManager::seq_len(int64_t id) const {
  auto it = seqs_.find(id);
  return it == seqs_.end() ? -1 : it->second.len;
}

int CacheManager::state_slot(int64_t id) const {
  auto it = seqs_.find(id);
  return it == seqs_.end() ? -1 : it->second.state_slot;
}

const std::vector<int32_t>* CacheManager::table(int64_t id, int group) const {
  auto it = seqs_.find(id);
  if (it == seqs_.end() || group < 0 || group >= (int)groups_.size()) return nullptr;
  return &it->second.tables[group];
}

int CacheManager::min_free_pages() const {
  if (groups_.empty()) return 1 << 30;  // nothing is paged: pages never limit
  int least = free_pages(0);
  for (size_t gi = 1; gi < groups_.size(); ++gi) least = std::min(least, free_pages((int)gi));
  return least;
}

std::vector<CopyOp> CacheManager::take_copies() {
  std::vector<CopyOp> out;
  out.swap(copies_);
  return out;
}

bool CacheManager::check_invariants(std::string* why) const {
  std::ostringstream msg;
  bool ok = true;
  for (size_t gi = 0; gi < groups_.size(); ++gi) {
    const Group& g = groups_[gi];
    std::vector<uint32_t> want(g.spec.num_pages, 0);
    for (auto& kv : seqs_)
      for (int32_t page : kv.second.tables[gi])
        if (page >= 0) {
          if (page >= g.spec.num_pages) { msg << "group " << gi << ": table entry " << page << " out of range; "; ok = false; continue; }
          ++want[page];
        }
    if (want != g.refs) { msg << "group " << gi << ": reference counts drifted; "; ok = false; }
    int idle = 0;
    for (uint32_t r : g.refs) idle += (r == 0);
    if (idle != free_pages((int)gi)) { msg << "group " << gi << ": free list drifted (" << idle << " idle, " << free_pages((int)gi) << " listed); "; ok = false; }
    std::vector<uint8_t> seen(g.spec.num_pages, 0);
    for (auto* list : {&g.free, &g.cached})
      for (int32_t page : *list) {
        if (page < 0 || page >= g.spec.num_pages || seen[page] || g.refs[page] != 0) { msg << "group " << gi << ": page " << page << " listed free twice or while held; "; ok = false; }
        else seen[page] = 1;
      }
    for (int32_t page : g.free)
      if (page >= 0 && page < g.spec.num_pages && g.has_hash[page]) { msg << "group " << gi << ": hashed page " << page << " on the plain free list; "; ok = false; }
    for (auto& kv : g.by_hash)
      if (!g.has_hash[kv.second] || g.page_hash[kv.second] != kv.first) { msg << "group " << gi << ": hash registration of page " << kv.second << " is stale; "; ok = false; }
  }
  if (num_state_slots_ > 0) {
    std::vector<uint8_t> seen(num_state_slots_, 0);
    for (int32_t s : free_slots_) {
      if (s < 0 || s >= num_state_slots_ || seen[s]) { msg << "state slot " << s << " free twice; "; ok = false; }
      else seen[s] = 1;
    }
    for (auto& kv : seqs_) {
      int32_t s = kv.second.state_slot;
      if (s < 0 || s >= num_state_slots_ || seen[s]) { msg << "state slot " << s << " held twice or while free; "; ok = false; }
      else seen[s] = 1;
    }
    for (int s = 0; s < num_state_slots_; ++s)
      if (!seen[s]) { msg << "state slot " << s << " lost; "; ok = false; }
  }
  if (why) *why = msg.str();
  return ok;
}

}  // namespace gb
