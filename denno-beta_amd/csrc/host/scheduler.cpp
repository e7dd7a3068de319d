#include "scheduler.h"

#include <algorithm>

namespace denno {

Scheduler::Scheduler(CacheManager* cache, int max_live, int max_batch_tokens, int prefill_chunk,
                     int policy, int max_positions)
    : cache_(cache), max_live_(std::min(max_live, cache->max_requests())),
      max_batch_tokens_(max_batch_tokens), prefill_chunk_(prefill_chunk), policy_(policy),
      max_positions_(max_positions), reserved_total_(cache->n_groups(), 0) {}

int Scheduler::add(int64_t rid, int prompt_len, int max_new) {
  if (reqs_.count(rid)) return kSchedDuplicate;
  if (prompt_len <= 0) return kEmptyPrompt;
  if (prompt_len > max_positions_) return kPromptTooLong;
  if (max_new < 0) max_new = 0;
  max_new = std::min(max_new, max_positions_ - prompt_len);
  // the last sampled token is never fed, so the cache holds at most prompt + max_new - 1 tokens
  int peak_len = prompt_len + std::max(0, max_new - 1);
  for (int g = 0; g < cache_->n_groups(); ++g) {
    if (cache_->group(g).kind != kPaged) continue;
    if (cache_->pages_peak(g, peak_len, prefill_chunk_) > cache_->group(g).n_pages) return kNeverFits;
  }
  Req r{rid, prompt_len, max_new, prompt_len, 0, 0, false, {}};
  reqs_.emplace(rid, r);
  waiting_.push_back(rid);
  return max_new;
}

int Scheduler::fit_tokens(const Req& r, int want) const {
  // the most tokens <= want whose pages every pool can give now
  int n = want;
  for (int g = 0; g < cache_->n_groups(); ++g) {
    const GroupSpec& s = cache_->group(g);
    if (s.kind != kPaged) continue;
    int blocks = r.running ? cache_->blocks(r.rid, g) : 0;
    int room = (blocks + cache_->free_pages(g)) * s.page_size - r.computed;
    n = std::min(n, room);
  }
  return std::max(n, 0);
}

bool Scheduler::try_admit(Req& r, int budget, int n_running_after) {
  if (static_cast<int>(running_.size()) >= max_live_) return false;
  int first = std::min({r.known - r.computed, prefill_chunk_, budget});
  if (first <= 0) return false;
  if (policy_ == kReserve) {
    int peak_len = r.prompt_len + std::max(0, r.max_new - 1);
    std::vector<int> need(cache_->n_groups(), 0);
    for (int g = 0; g < cache_->n_groups(); ++g) {
      if (cache_->group(g).kind != kPaged) continue;
      need[g] = cache_->pages_peak(g, peak_len, prefill_chunk_);
      if (reserved_total_[g] + need[g] > cache_->group(g).n_pages) return false;
    }
    r.reserved = need;
  } else {
    // leave a page for every request that is already running: each may need one soon
    for (int g = 0; g < cache_->n_groups(); ++g) {
      if (cache_->group(g).kind != kPaged) continue;
      int need = cache_->pages_needed(-1, 0, first, g);
      if (need + (running_.empty() ? 0 : n_running_after) > cache_->free_pages(g)) return false;
    }
  }
  int slot = cache_->add(r.rid);
  if (slot < 0) {
    r.reserved.clear();
    return false;
  }
  if (policy_ == kReserve)
    for (int g = 0; g < cache_->n_groups(); ++g) reserved_total_[g] += r.reserved[g];
  r.running = true;
  return true;
}

void Scheduler::preempt(size_t i, std::vector<int64_t>* preempted) {
  int64_t rid = running_[i];
  Req& r = reqs_.at(rid);
  cache_->release(rid);
  r.computed = 0;
  r.running = false;
  running_.erase(running_.begin() + static_cast<long>(i));
  waiting_.push_front(rid);
  if (preempted) preempted->push_back(rid);
}

int Scheduler::schedule(std::vector<StepEntry>* out, std::vector<int64_t>* preempted) {
  out->clear();
  if (preempted) preempted->clear();
  std::vector<int64_t> just_preempted;
  for (;;) {
    out->clear();
    int budget = max_batch_tokens_;
    bool retry = false;
    // 1. decodes, oldest first
    for (size_t i = 0; i < running_.size() && !retry; ++i) {
      Req& r = reqs_.at(running_[i]);
      if (r.known - r.computed != 1 || r.generated == 0) continue;
      if (budget <= 0) break;
      while (cache_->reserve(r.rid, r.computed + 1) == kOutOfPages) {
        // kReserve never comes here.  The youngest gives way, never one older than r.
        size_t victim = running_.size() - 1;
        bool self = victim == i;
        // entries already planned for the victim are dropped with the retry
        preempt(victim, &just_preempted);
        retry = true;
        if (self) break;
      }
      if (retry) break;
      out->push_back({r.rid, r.computed, 1, 1});
      budget -= 1;
    }
    if (retry) continue;
    // 2. prompts under way (and recomputations), oldest first
    for (size_t i = 0; i < running_.size(); ++i) {
      Req& r = reqs_.at(running_[i]);
      int remaining = r.known - r.computed;
      if (remaining <= 0 || (remaining == 1 && r.generated > 0)) continue;
      int want = std::min({remaining, prefill_chunk_, budget});
      if (want <= 0) continue;
      int n = policy_ == kReserve ? want : fit_tokens(r, want);
      if (n <= 0) continue;
      if (cache_->reserve(r.rid, r.computed + n) != kOk) continue;
      out->push_back({r.rid, r.computed, n, n == remaining ? 1 : 0});
      budget -= n;
    }
    // 3. admissions, first come first served; a request preempted in this call waits a step
    while (!waiting_.empty() && budget > 0) {
      int64_t rid = waiting_.front();
      if (std::find(just_preempted.begin(), just_preempted.end(), rid) != just_preempted.end()) break;
      Req& r = reqs_.at(rid);
      if (!try_admit(r, budget, static_cast<int>(running_.size()))) break;
      waiting_.pop_front();
      running_.push_back(rid);
      int remaining = r.known - r.computed;
      int want = std::min({remaining, prefill_chunk_, budget});
      int n = policy_ == kReserve ? want : fit_tokens(r, want);
      if (n > 0 && cache_->reserve(rid, r.computed + n) == kOk) {
        out->push_back({rid, r.computed, n, n == remaining ? 1 : 0});
        budget -= n;
      }
    }
    if (out->empty() && running_.size() > 1 && policy_ == kPreempt) {
      // every running request is stuck in mid-prompt with the pools full: the youngest gives way
      preempt(running_.size() - 1, &just_preempted);
      continue;
    }
    break;
  }
  if (preempted) *preempted = just_preempted;
  return static_cast<int>(out->size());
}

int Scheduler::step_done(int64_t rid, int count) {
  auto it = reqs_.find(rid);
  if (it == reqs_.end()) return kSchedUnknown;
  Req& r = it->second;
  if (!r.running || r.computed + count > r.known) return kSchedBadState;
  r.computed += count;
  int rc = cache_->commit(rid, r.computed);
  return rc == kOk ? static_cast<int>(kSchedOk) : rc;
}

int Scheduler::token_sampled(int64_t rid) {
  auto it = reqs_.find(rid);
  if (it == reqs_.end()) return kSchedUnknown;
  Req& r = it->second;
  if (r.computed != r.known || r.generated >= r.max_new) return kSchedBadState;
  r.known += 1;
  r.generated += 1;
  return r.generated >= r.max_new ? 1 : 0;
}

int Scheduler::steps_done(const int64_t* rids, const int* counts, int n, int* failed) {
  for (int i = 0; i < n; ++i) {
    int rc = step_done(rids[i], counts[i]);
    if (rc < 0) {
      *failed = i;
      return rc;
    }
  }
  return kSchedOk;
}

int Scheduler::tokens_sampled(const int64_t* rids, int n, int* last, int* failed) {
  for (int i = 0; i < n; ++i) {
    int rc = token_sampled(rids[i]);
    if (rc < 0) {
      *failed = i;
      return rc;
    }
    last[i] = rc;
  }
  return kSchedOk;
}

int Scheduler::finish(int64_t rid) {
  auto it = reqs_.find(rid);
  if (it == reqs_.end()) return kSchedUnknown;
  Req& r = it->second;
  if (r.running) {
    cache_->release(rid);
    running_.erase(std::find(running_.begin(), running_.end(), rid));
    if (policy_ == kReserve)
      for (size_t g = 0; g < r.reserved.size(); ++g) reserved_total_[g] -= r.reserved[g];
  } else {
    waiting_.erase(std::find(waiting_.begin(), waiting_.end(), rid));
  }
  reqs_.erase(it);
  return kSchedOk;
}

int Scheduler::abort_step(const std::vector<int64_t>& rids) {
  for (int64_t rid : rids) finish(rid);
  return kSchedOk;
}

int Scheduler::known(int64_t rid) const {
  auto it = reqs_.find(rid);
  return it == reqs_.end() ? static_cast<int>(kSchedUnknown) : it->second.known;
}
int Scheduler::computed(int64_t rid) const {
  auto it = reqs_.find(rid);
  return it == reqs_.end() ? static_cast<int>(kSchedUnknown) : it->second.computed;
}
int Scheduler::generated(int64_t rid) const {
  auto it = reqs_.find(rid);
  return it == reqs_.end() ? static_cast<int>(kSchedUnknown) : it->second.generated;
}

}  // namespace denno
