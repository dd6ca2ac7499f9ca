// Paged cache bookkeeping on the host: which pages of which pool belong to which
// request.  It owns no device memory; the engine keeps one device tensor of pages
// per layer and indexes it with the page numbers handed out here.
//
// Behaviour follows the reference's KvCache (crates/glassbox-core/src/kv.rs):
// fixed-size pages, a block table per request, reference counts, prefix sharing
// through a hash chain over full pages, copy-on-write of a shared partial page,
// and a "cached" list of unreferenced pages that still carry a prefix hash.
// Added here: several page groups (layers whose mixers need all keys, or only a
// window of them, each with a pool of its own) and fixed-size state slots.
#pragma once
#include <cstdint>
#include <string>
#include <unordered_map>
#include <vector>

namespace gb {

enum GroupKind : int { kFull = 0, kWindow = 1 };

struct GroupSpec {
  int kind = kFull;
  int window = 0;      // kWindow: a query at position p reads keys p-window+1 .. p
  int num_pages = 0;
};

struct CopyOp {        // device work the engine must do before the next step; dropped if dst is given back first
  int group;           // >= 0: copy page src -> dst in every layer of the group
  int src;             //  -1 : copy state slot src -> dst
  int dst;
};

class CacheManager {
 public:
  CacheManager(int page_size, std::vector<GroupSpec> groups, int num_state_slots, bool share_prefixes);

  // A new request.  Returns how many prompt tokens are already in the cache
  // (kv.rs:135-157: a multiple of the page size and never the whole prompt),
  // -1 if the id exists, -2 if no state slot is free.
  int add_seq(int64_t id, const int32_t* prompt, int n);
  // Room for positions len .. len+n.  0 = done, 1 = out of pages (nothing
  // changed, kv.rs:161-187), -1 = unknown id.
  int reserve(int64_t id, int n);
  // Positions up to len+n are written (kv.rs:205-233).  Full pages are hashed;
  // pages a window has passed are given back.
  int commit(int64_t id, const int32_t* tokens, int n);
  int truncate(int64_t id, int len);             // kv.rs:237-257
  int fork(int64_t parent, int64_t child);       // kv.rs:260-266
  int remove_seq(int64_t id);                    // kv.rs:268-274

  bool has_seq(int64_t id) const { return seqs_.count(id) != 0; }
  int seq_len(int64_t id) const;
  int state_slot(int64_t id) const;
  const std::vector<int32_t>* table(int64_t id, int group) const;
  int page_size() const { return page_size_; }
  int num_groups() const { return (int)groups_.size(); }
  int num_pages(int g) const { return groups_[g].spec.num_pages; }
  int free_pages(int g) const { return (int)(groups_[g].free.size() + groups_[g].cached.size()); }
  int used_pages(int g) const { return num_pages(g) - free_pages(g); }
  int min_free_pages() const;
  int ref_count(int g, int page) const { return groups_[g].refs[page]; }
  int free_state_slots() const { return (int)free_slots_.size(); }
  int num_seqs() const { return (int)seqs_.size(); }
  bool share_prefixes() const { return share_; }
  // How many pages `reserve(id, n)` would have to take from each pool's free
  // list, summed over groups that limit it (the largest demand over groups).
  int pages_needed(int64_t id, int n) const;

  std::vector<CopyOp> take_copies();
  // refs == table entries pointing at a page; idle pages == free + cached;
  // no page on a free list twice; every state slot held once (kv.rs:278-288).
  bool check_invariants(std::string* why) const;

 private:
  struct Group {
    GroupSpec spec;
    std::vector<uint32_t> refs;
    std::vector<int32_t> free;                 // LIFO, page 0 handed out first
    std::vector<int32_t> cached;               // idle pages that keep a prefix hash, oldest first
    std::unordered_map<uint64_t, int32_t> by_hash;
    std::vector<uint64_t> page_hash;
    std::vector<uint8_t> has_hash;
  };
  struct Seq {
    std::vector<std::vector<int32_t>> tables;  // [group][logical page] -> page or -1 (given back)
    int len = 0;
    std::vector<int32_t> tokens;
    int state_slot = -1;
  };

  int alloc(Group& g);
  void release(Group& g, int32_t page);
  void retain(Group& g, int32_t page);
  void drop_copies_into(int group, int32_t dst);  // group -1: a state slot
  int need_in_group(const Seq& s, int gi, int n) const;

  int page_size_;
  std::vector<Group> groups_;
  std::unordered_map<int64_t, Seq> seqs_;
  std::vector<int32_t> free_slots_;
  int num_state_slots_;
  bool share_;
  std::vector<CopyOp> copies_;
};

uint64_t chain_hash(uint64_t prev, const int32_t* tokens, int n);  // kv.rs:45-55

}  // namespace gb
