// The scheduler: which requests run in the next step, and how many of their tokens.
//
// The reference admits up to four sessions, runs a new session's whole prompt alone and
// ahead of everything else, and otherwise decodes all sessions together
// (crates/denno-server/src/scheduler.rs:65, 311-324, 351-419); it reserves prompt +
// max_tokens at admission, so it never runs out in mid-run (crates/denno-engine/src/engine.rs:
// 526-588).  Here a step is a mixed batch under a token budget: every running request whose
// next token is known decodes (one token each), then prompts go on in portions.
//
// A request is a count of known tokens (prompt + sampled) and a count of tokens in the
// cache; feeding goes on until they are equal, then a token is sampled and one more is
// known.  A decode is the case "one token missing".
//
// When pages run out there are two policies.  kReserve: as the reference, a request is
// admitted only if its peak need (prompt + max_new) can be set aside, so running requests
// never lack a page; others wait.  kPreempt: pages are taken step by step; when a running
// request cannot get its page, the youngest running request gives everything back and
// returns to the head of the queue, to be recomputed from its known tokens later.  The oldest
// is never preempted for a younger one, so the oldest always goes on.
#pragma once
#include <cstddef>
#include <cstdint>
#include <deque>
#include <unordered_map>
#include <vector>

#include "cache_manager.h"

namespace denno {

enum SchedPolicy : int { kPreempt = 0, kReserve = 1 };

enum SchedStatus : int {
  kSchedOk = 0,
  kEmptyPrompt = -10,
  kPromptTooLong = -11,   // the prompt fills the context: no position is left for a new token
  kNeverFits = -12,       // even alone, the request needs more pages than a pool has
  kSchedDuplicate = -13,
  kSchedUnknown = -14,
  kSchedBadState = -15,
};

struct StepEntry {
  int64_t rid;
  int start;     // tokens in the cache before the step
  int count;     // tokens to feed
  int samples;   // 1: the step brings the request to its last known token, so its last row is sampled
};

class Scheduler {
 public:
  Scheduler(CacheManager* cache, int max_live, int max_batch_tokens, int prefill_chunk, int policy,
            int max_positions);

  // max_new is clamped to max_positions - prompt_len, as the reference clamps max_tokens
  // (crates/denno-engine/src/engine.rs:865-881); the clamped value is returned (>= 0), or a SchedStatus
  int add(int64_t rid, int prompt_len, int max_new);
  int schedule(std::vector<StepEntry>* out, std::vector<int64_t>* preempted);
  int step_done(int64_t rid, int count);   // the step ran: count more tokens are in the cache
  int token_sampled(int64_t rid);          // -> 1 if that token was the request's last (length), else 0
  // the same for all entries of a step in one call each; last[i] as token_sampled returns it.  On a failure
  // *failed is the entry's index and the entries before it have been done.
  int steps_done(const int64_t* rids, const int* counts, int n, int* failed);
  int tokens_sampled(const int64_t* rids, int n, int* last, int* failed);
  int finish(int64_t rid);                 // pages and slot go back (running or waiting)
  int abort_step(const std::vector<int64_t>& rids);   // a failed step: its requests are dropped, pages back

  int n_waiting() const { return static_cast<int>(waiting_.size()); }
  int n_running() const { return static_cast<int>(running_.size()); }
  int known(int64_t rid) const;
  int computed(int64_t rid) const;
  int generated(int64_t rid) const;

 private:
  struct Req {
    int64_t rid;
    int prompt_len;
    int max_new;
    int known;       // prompt + sampled tokens
    int computed;    // tokens in the cache
    int generated;
    bool running;
    std::vector<int> reserved;   // kReserve: pages set aside per group
  };
  bool try_admit(Req& r, int budget, int n_running_after);
  void preempt(size_t running_index, std::vector<int64_t>* preempted);
  int fit_tokens(const Req& r, int want) const;

  CacheManager* cache_;
  int max_live_, max_batch_tokens_, prefill_chunk_, policy_, max_positions_;
  std::unordered_map<int64_t, Req> reqs_;
  std::deque<int64_t> waiting_;
  std::vector<int64_t> running_;           // in order of admission, oldest first
  std::vector<int> reserved_total_;        // kReserve
};

}  // namespace denno
