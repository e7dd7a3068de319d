// Cache bookkeeping: pages of keys and values with one block table per request and
// group, and slots for per-request state of fixed size.  Host-only; the device
// tensors that the pages and slots index are owned by the caller.
//
// The reference keeps one contiguous, growable buffer per request and layer
// (crates/denno-engine/src/kv_cache.rs:17-25, 175-202) and guards a slot's release with a
// lease id (crates/denno-engine/src/engine.rs:751-769).  Here the unit is a page; a group
// of layers that needs all keys and a group that needs a window of them draw from pools
// of their own; a slot's generation plays the lease's part.
#pragma once
#include <cstddef>
#include <cstdint>
#include <unordered_map>
#include <vector>

namespace denno {

enum GroupKind : int { kPaged = 0, kState = 1 };

enum CacheStatus : int {
  kOk = 0,
  kNoSlot = -1,        // every request slot is taken
  kDuplicate = -2,     // the request id is live already
  kUnknown = -3,       // no live request has this id (a stale release is this, and changes nothing)
  kOutOfPages = -4,    // a pool cannot give the pages asked for; nothing was changed
  kBadArgument = -5,
  kCorrupt = -6,       // check() found a page lost, held twice or free and held
};

struct GroupSpec {
  int kind;        // GroupKind
  int n_pages;     // pool size (paged groups)
  int page_size;   // tokens in a page
  int window;      // 0: every key is kept; W > 0: a query at position p reads keys in (p - W, p]
};

// What a live request keeps beside its pages, in its slot: a record of fixed size, zero when the slot
// is given out.  The reference keeps the position in its cache object and the sampler's generator in
// the session (crates/denno-engine/src/kv_cache.rs:21, 133-135; engine.rs:251).  The generator here is
// counter-based: its whole state is the seed and the count of numbers drawn.
struct SlotState {
  int32_t num_computed;   // tokens in the cache = the next token's position
  int32_t last_token;     // the token sampled last, -1 before the first
  uint64_t rng_seed;
  uint64_t rng_drawn;     // numbers drawn from the generator so far
};

class CacheManager {
 public:
  CacheManager(const std::vector<GroupSpec>& groups, int max_requests);

  int add(int64_t rid);                       // -> slot >= 0, or a CacheStatus < 0
  int release(int64_t rid);                   // gives back pages and slot
  int reserve(int64_t rid, int new_len);      // pages for positions [len, new_len) in every paged group
  int commit(int64_t rid, int new_len);       // len = new_len; pages that a window has passed go back
  int length(int64_t rid) const;              // tokens committed, or kUnknown
  int slot(int64_t rid) const;
  // the request's slot record; 0 if the id is not live.  set_rng: at admission (a request that was
  // preempted brings the count it had); note_sampled: one more number drawn, `token` sampled with it
  const SlotState* state(int64_t rid) const;
  int set_rng(int64_t rid, uint64_t seed, uint64_t drawn);
  int note_sampled(int64_t rid, int32_t token);
  // the same in two halves, for a step's requests at once: a number was drawn for each (when the sampling
  // kernel is launched), and later the tokens that it gave are known; ids that are no longer live are skipped
  void note_drawn_step(const int64_t* rids, int n);
  void note_tokens_step(const int64_t* rids, const int32_t* tokens, int n);
  // seeds and counts of a step's requests in one call; on a failure *failed is the entry's index
  int rng_states(const int64_t* rids, int n, uint64_t* seeds, uint64_t* drawn, int* failed) const;
  int64_t generation(int slot) const;         // bumped each time the slot is given out
  int block_table(int64_t rid, int group, int32_t* out, int cap) const;   // -> blocks; -1 marks a page given back
  int free_pages(int group) const;
  int pages_held(int64_t rid, int group) const;
  int blocks(int64_t rid, int group) const;   // entries of the block table, given back or not
  // pages that reserve(rid, new_len) would take from `group` (rid < 0: a request not yet added, of length from_len)
  int pages_needed(int64_t rid, int from_len, int new_len, int group) const;
  // most pages that a request of `total_len` tokens, fed in portions of at most `chunk`, holds at once
  int pages_peak(int group, int total_len, int chunk) const;

  // The same for all requests of a step in one call each (a step of 64 single tokens is otherwise
  // some hundred calls across the language boundary).  On a failure *failed is the entry's index.
  int lengths(const int64_t* rids, int n, int* out, int* failed) const;
  // pages for every entry's tokens, entry after entry; entries before a failing one keep theirs
  int reserve_step(const int64_t* rids, const int* new_lens, int n, int* slots_out, int* failed);
  int commit_step(const int64_t* rids, const int* new_lens, int n, int* failed);
  int max_blocks(int group, const int64_t* rids, int n) const;      // the longest block table, or < 0
  // The tables that the kernels read for one group: block_tables [bt_rows, max_blocks] (row i: entry
  // i's; -1 where there is no page, and in rows n .. bt_rows - 1) and slot_map [sm_len] (token j of
  // entry i at sum(counts[:i]) + j: page * page_size + offset of position starts[i] + j; -1 beyond
  // the entries' tokens).  kBadArgument if a table or the map is too small or a token's page was
  // given back.
  int step_tables(int group, const int64_t* rids, const int* starts, const int* counts, int n, int bt_rows,
                  int max_blocks, int32_t* block_tables, int32_t* slot_map, int sm_len, int* failed) const;

  int live() const { return static_cast<int>(by_rid_.size()); }
  int n_groups() const { return static_cast<int>(groups_.size()); }
  const GroupSpec& group(int g) const { return groups_[g]; }
  int max_requests() const { return static_cast<int>(slot_rid_.size()); }
  int check() const;                          // kOk, or kCorrupt
  int64_t reuse_count(int group) const { return reuse_[group]; }  // pages given out that were held before

 private:
  struct Request {
    int slot;                                  // index of its SlotState (the position lives there)
    std::vector<std::vector<int32_t>> tables;  // [group][block] -> page, -1 once given back
    std::vector<int> first_live;               // [group] first block that is still held
  };
  int first_needed_block(int g, int len) const;

  std::vector<GroupSpec> groups_;
  std::vector<std::vector<int32_t>> free_;     // [group] stack of free pages
  std::vector<std::vector<uint8_t>> used_before_;
  std::vector<int64_t> reuse_;
  std::vector<int64_t> slot_rid_;              // [slot] rid, or -1
  std::vector<int64_t> slot_gen_;
  std::vector<SlotState> slot_state_;          // [slot]
  std::vector<int> free_slots_;
  std::unordered_map<int64_t, Request> by_rid_;
};

}  // namespace denno
