#include "cache_manager.h"

#include <algorithm>

namespace denno {

CacheManager::CacheManager(const std::vector<GroupSpec>& groups, int max_requests)
    : groups_(groups), free_(groups.size()), used_before_(groups.size()), reuse_(groups.size(), 0),
      slot_rid_(max_requests, -1), slot_gen_(max_requests, 0),
      slot_state_(max_requests, SlotState{0, -1, 0, 0}) {
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].kind != kPaged) continue;
    // a stack whose top is page 0, so a fresh pool hands pages out in ascending order
    for (int p = groups_[g].n_pages - 1; p >= 0; --p) free_[g].push_back(p);
    used_before_[g].assign(groups_[g].n_pages, 0);
  }
  for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);
}

int CacheManager::add(int64_t rid) {
  if (rid < 0) return kBadArgument;
  if (by_rid_.count(rid)) return kDuplicate;
  if (free_slots_.empty()) return kNoSlot;
  Request r;
  r.slot = free_slots_.back();
  free_slots_.pop_back();
  slot_state_[r.slot] = SlotState{0, -1, 0, 0};
  r.tables.resize(groups_.size());
  r.first_live.assign(groups_.size(), 0);
  slot_rid_[r.slot] = rid;
  slot_gen_[r.slot] += 1;
  int slot = r.slot;
  by_rid_.emplace(rid, std::move(r));
  return slot;
}

int CacheManager::release(int64_t rid) {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  Request& r = it->second;
  for (size_t g = 0; g < groups_.size(); ++g)
    for (int32_t p : r.tables[g])
      if (p >= 0) free_[g].push_back(p);
  slot_rid_[r.slot] = -1;
  free_slots_.push_back(r.slot);
  by_rid_.erase(it);
  return kOk;
}

int CacheManager::first_needed_block(int g, int len) const {
  // the next query stands at position >= len and reads keys > len - window
  const GroupSpec& s = groups_[g];
  if (s.window <= 0) return 0;
  int first_key = len - s.window + 1;
  return first_key <= 0 ? 0 : first_key / s.page_size;
}

int CacheManager::pages_needed(int64_t rid, int from_len, int new_len, int g) const {
  if (g < 0 || g >= n_groups() || groups_[g].kind != kPaged) return 0;
  int have = 0;
  if (rid >= 0) {
    auto it = by_rid_.find(rid);
    if (it == by_rid_.end()) return kUnknown;
    have = static_cast<int>(it->second.tables[g].size());
  } else {
    have = (from_len + groups_[g].page_size - 1) / groups_[g].page_size;
  }
  int want = (new_len + groups_[g].page_size - 1) / groups_[g].page_size;
  return std::max(0, want - have);
}

int CacheManager::pages_peak(int g, int total_len, int chunk) const {
  if (g < 0 || g >= n_groups() || groups_[g].kind != kPaged) return 0;
  const GroupSpec& s = groups_[g];
  int all = (total_len + s.page_size - 1) / s.page_size;
  if (s.window <= 0) return all;
  // window keys before the portion, the portion itself, and one page of slack at each edge
  int span = (s.window + std::max(chunk, 1) + s.page_size - 1) / s.page_size + 1;
  return std::min(all, span);
}

int CacheManager::reserve(int64_t rid, int new_len) {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  Request& r = it->second;
  if (new_len < slot_state_[r.slot].num_computed) return kBadArgument;
  std::vector<int> need(groups_.size(), 0);
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].kind != kPaged) continue;
    int want = (new_len + groups_[g].page_size - 1) / groups_[g].page_size;
    need[g] = std::max(0, want - static_cast<int>(r.tables[g].size()));
    if (need[g] > static_cast<int>(free_[g].size())) return kOutOfPages;
  }
  for (size_t g = 0; g < groups_.size(); ++g) {
    for (int i = 0; i < need[g]; ++i) {
      int32_t p = free_[g].back();
      free_[g].pop_back();
      if (used_before_[g][p]) reuse_[g] += 1;
      used_before_[g][p] = 1;
      r.tables[g].push_back(p);
    }
  }
  return kOk;
}

int CacheManager::commit(int64_t rid, int new_len) {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  Request& r = it->second;
  if (new_len < slot_state_[r.slot].num_computed) return kBadArgument;
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].kind != kPaged) continue;
    int blocks = static_cast<int>(r.tables[g].size());
    if (new_len > blocks * groups_[g].page_size) return kBadArgument;   // commit without reserve
  }
  slot_state_[r.slot].num_computed = new_len;
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].kind != kPaged) continue;
    int first = std::min(first_needed_block(static_cast<int>(g), new_len),
                         static_cast<int>(r.tables[g].size()));
    for (int b = r.first_live[g]; b < first; ++b) {
      if (r.tables[g][b] >= 0) {
        free_[g].push_back(r.tables[g][b]);
        r.tables[g][b] = -1;
      }
    }
    r.first_live[g] = std::max(r.first_live[g], first);
  }
  return kOk;
}

int CacheManager::lengths(const int64_t* rids, int n, int* out, int* failed) const {
  for (int i = 0; i < n; ++i) {
    auto it = by_rid_.find(rids[i]);
    if (it == by_rid_.end()) {
      *failed = i;
      return kUnknown;
    }
    out[i] = slot_state_[it->second.slot].num_computed;
  }
  return kOk;
}

int CacheManager::reserve_step(const int64_t* rids, const int* new_lens, int n, int* slots_out, int* failed) {
  for (int i = 0; i < n; ++i) {
    int rc = reserve(rids[i], new_lens[i]);
    if (rc != kOk) {
      *failed = i;
      return rc;
    }
    slots_out[i] = by_rid_.find(rids[i])->second.slot;
  }
  return kOk;
}

int CacheManager::commit_step(const int64_t* rids, const int* new_lens, int n, int* failed) {
  for (int i = 0; i < n; ++i) {
    int rc = commit(rids[i], new_lens[i]);
    if (rc != kOk) {
      *failed = i;
      return rc;
    }
  }
  return kOk;
}

int CacheManager::max_blocks(int g, const int64_t* rids, int n) const {
  if (g < 0 || g >= n_groups()) return kBadArgument;
  int most = 0;
  for (int i = 0; i < n; ++i) {
    auto it = by_rid_.find(rids[i]);
    if (it == by_rid_.end()) return kUnknown;
    most = std::max(most, static_cast<int>(it->second.tables[g].size()));
  }
  return most;
}

int CacheManager::step_tables(int g, const int64_t* rids, const int* starts, const int* counts, int n, int bt_rows,
                              int max_blocks, int32_t* block_tables, int32_t* slot_map, int sm_len,
                              int* failed) const {
  if (g < 0 || g >= n_groups() || groups_[g].kind != kPaged || n > bt_rows || max_blocks < 1) return kBadArgument;
  const int ps = groups_[g].page_size;
  std::fill(block_tables, block_tables + static_cast<size_t>(bt_rows) * max_blocks, -1);
  std::fill(slot_map, slot_map + sm_len, -1);
  int row = 0;
  for (int i = 0; i < n; ++i) {
    *failed = i;
    auto it = by_rid_.find(rids[i]);
    if (it == by_rid_.end()) return kUnknown;
    const auto& t = it->second.tables[g];
    if (static_cast<int>(t.size()) > max_blocks || starts[i] < 0 || counts[i] < 0 || row + counts[i] > sm_len)
      return kBadArgument;
    std::copy(t.begin(), t.end(), block_tables + static_cast<size_t>(i) * max_blocks);
    for (int j = 0; j < counts[i]; ++j) {
      const int pos = starts[i] + j, blk = pos / ps;
      if (blk >= static_cast<int>(t.size()) || t[blk] < 0) return kBadArgument;     // no page, or given back
      slot_map[row + j] = t[blk] * ps + pos % ps;
    }
    row += counts[i];
  }
  return kOk;
}

int CacheManager::length(int64_t rid) const {
  auto it = by_rid_.find(rid);
  return it == by_rid_.end() ? static_cast<int>(kUnknown) : slot_state_[it->second.slot].num_computed;
}

int CacheManager::slot(int64_t rid) const {
  auto it = by_rid_.find(rid);
  return it == by_rid_.end() ? static_cast<int>(kUnknown) : it->second.slot;
}

const SlotState* CacheManager::state(int64_t rid) const {
  auto it = by_rid_.find(rid);
  return it == by_rid_.end() ? nullptr : &slot_state_[it->second.slot];
}

int CacheManager::set_rng(int64_t rid, uint64_t seed, uint64_t drawn) {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  slot_state_[it->second.slot].rng_seed = seed;
  slot_state_[it->second.slot].rng_drawn = drawn;
  return kOk;
}

int CacheManager::note_sampled(int64_t rid, int32_t token) {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  slot_state_[it->second.slot].rng_drawn += 1;
  slot_state_[it->second.slot].last_token = token;
  return kOk;
}

void CacheManager::note_drawn_step(const int64_t* rids, int n) {
  for (int i = 0; i < n; ++i) {
    auto it = by_rid_.find(rids[i]);
    if (it != by_rid_.end()) slot_state_[it->second.slot].rng_drawn += 1;
  }
}

void CacheManager::note_tokens_step(const int64_t* rids, const int32_t* tokens, int n) {
  for (int i = 0; i < n; ++i) {
    auto it = by_rid_.find(rids[i]);
    if (it != by_rid_.end()) slot_state_[it->second.slot].last_token = tokens[i];
  }
}

int CacheManager::rng_states(const int64_t* rids, int n, uint64_t* seeds, uint64_t* drawn, int* failed) const {
  for (int i = 0; i < n; ++i) {
    auto it = by_rid_.find(rids[i]);
    if (it == by_rid_.end()) {
      *failed = i;
      return kUnknown;
    }
    seeds[i] = slot_state_[it->second.slot].rng_seed;
    drawn[i] = slot_state_[it->second.slot].rng_drawn;
  }
  return kOk;
}

int64_t CacheManager::generation(int slot) const {
  if (slot < 0 || slot >= max_requests()) return -1;
  return slot_gen_[slot];
}

int CacheManager::block_table(int64_t rid, int g, int32_t* out, int cap) const {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  if (g < 0 || g >= n_groups()) return kBadArgument;
  const auto& t = it->second.tables[g];
  int n = static_cast<int>(t.size());
  if (n > cap) return kBadArgument;
  std::copy(t.begin(), t.end(), out);
  return n;
}

int CacheManager::free_pages(int g) const {
  if (g < 0 || g >= n_groups()) return kBadArgument;
  return static_cast<int>(free_[g].size());
}

int CacheManager::pages_held(int64_t rid, int g) const {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  if (g < 0 || g >= n_groups()) return kBadArgument;
  int n = 0;
  for (int32_t p : it->second.tables[g]) n += p >= 0;
  return n;
}

int CacheManager::blocks(int64_t rid, int g) const {
  auto it = by_rid_.find(rid);
  if (it == by_rid_.end()) return kUnknown;
  if (g < 0 || g >= n_groups()) return kBadArgument;
  return static_cast<int>(it->second.tables[g].size());
}

int CacheManager::check() const {
  for (size_t g = 0; g < groups_.size(); ++g) {
    if (groups_[g].kind != kPaged) continue;
    std::vector<int> seen(groups_[g].n_pages, 0);
    for (int32_t p : free_[g]) {
      if (p < 0 || p >= groups_[g].n_pages) return kCorrupt;
      seen[p] += 1;
    }
    for (const auto& kv : by_rid_)
      for (int32_t p : kv.second.tables[g]) {
        if (p == -1) continue;
        if (p < 0 || p >= groups_[g].n_pages) return kCorrupt;
        seen[p] += 1;
      }
    for (int c : seen)
      if (c != 1) return kCorrupt;   // 0: lost; 2: held twice, freed twice, or free and held
  }
  std::vector<int> slots(slot_rid_.size(), 0);
  for (int s : free_slots_) {
    if (s < 0 || s >= max_requests() || slot_rid_[s] != -1) return kCorrupt;
    slots[s] += 1;
  }
  for (const auto& kv : by_rid_) {
    int s = kv.second.slot;
    if (s < 0 || s >= max_requests() || slot_rid_[s] != kv.first) return kCorrupt;
    slots[s] += 1;
  }
  for (int c : slots)
    if (c != 1) return kCorrupt;
  return kOk;
}

}  // namespace denno
