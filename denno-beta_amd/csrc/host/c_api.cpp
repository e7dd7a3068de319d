// C ABI of the host core, for ctypes.  Every function returns a status or a count;
// none throws across the boundary.
#include <cstddef>
#include <cstdint>
#include <new>
#include <vector>

#include "cache_manager.h"
#include "scheduler.h"

using denno::CacheManager;
using denno::GroupSpec;
using denno::Scheduler;
using denno::StepEntry;

extern "C" {

void* dn_cache_create(int n_groups, const int* kinds, const int* n_pages, const int* page_size,
                      const int* window, int max_requests) {
  if (n_groups < 0 || max_requests < 1) return nullptr;
  std::vector<GroupSpec> g(n_groups);
  for (int i = 0; i < n_groups; ++i) {
    g[i] = GroupSpec{kinds[i], n_pages[i], page_size[i], window[i]};
    if (kinds[i] == denno::kPaged && (n_pages[i] < 1 || page_size[i] < 1 || window[i] < 0)) return nullptr;
  }
  return new (std::nothrow) CacheManager(g, max_requests);
}
void dn_cache_destroy(void* c) { delete static_cast<CacheManager*>(c); }
int dn_cache_add(void* c, int64_t rid) { return static_cast<CacheManager*>(c)->add(rid); }
int dn_cache_release(void* c, int64_t rid) { return static_cast<CacheManager*>(c)->release(rid); }
int dn_cache_reserve(void* c, int64_t rid, int n) { return static_cast<CacheManager*>(c)->reserve(rid, n); }
int dn_cache_commit(void* c, int64_t rid, int n) { return static_cast<CacheManager*>(c)->commit(rid, n); }
int dn_cache_length(void* c, int64_t rid) { return static_cast<CacheManager*>(c)->length(rid); }
int dn_cache_slot(void* c, int64_t rid) { return static_cast<CacheManager*>(c)->slot(rid); }
// out: num_computed, last_token, then the seed and the count of numbers drawn as two 32-bit halves each (low first)
int dn_cache_state(void* c, int64_t rid, int64_t* out) {
  const denno::SlotState* s = static_cast<CacheManager*>(c)->state(rid);
  if (!s) return denno::kUnknown;
  out[0] = s->num_computed;
  out[1] = s->last_token;
  out[2] = static_cast<int64_t>(s->rng_seed & 0xffffffffu);
  out[3] = static_cast<int64_t>(s->rng_seed >> 32);
  out[4] = static_cast<int64_t>(s->rng_drawn & 0xffffffffu);
  out[5] = static_cast<int64_t>(s->rng_drawn >> 32);
  return denno::kOk;
}
int dn_cache_set_rng(void* c, int64_t rid, uint64_t seed, uint64_t drawn) {
  return static_cast<CacheManager*>(c)->set_rng(rid, seed, drawn);
}
int dn_cache_note_sampled(void* c, int64_t rid, int token) {
  return static_cast<CacheManager*>(c)->note_sampled(rid, token);
}
void dn_cache_note_drawn_step(void* c, const int64_t* rids, int n) {
  static_cast<CacheManager*>(c)->note_drawn_step(rids, n);
}
void dn_cache_note_tokens_step(void* c, const int64_t* rids, const int32_t* tokens, int n) {
  static_cast<CacheManager*>(c)->note_tokens_step(rids, tokens, n);
}
int dn_cache_rng_states(void* c, const int64_t* rids, int n, uint64_t* seeds, uint64_t* drawn, int* failed) {
  return static_cast<CacheManager*>(c)->rng_states(rids, n, seeds, drawn, failed);
}
int64_t dn_cache_generation(void* c, int slot) { return static_cast<CacheManager*>(c)->generation(slot); }
int dn_cache_block_table(void* c, int64_t rid, int g, int32_t* out, int cap) {
  return static_cast<CacheManager*>(c)->block_table(rid, g, out, cap);
}
int dn_cache_blocks(void* c, int64_t rid, int g) { return static_cast<CacheManager*>(c)->blocks(rid, g); }
int dn_cache_free_pages(void* c, int g) { return static_cast<CacheManager*>(c)->free_pages(g); }
int dn_cache_pages_held(void* c, int64_t rid, int g) { return static_cast<CacheManager*>(c)->pages_held(rid, g); }
int dn_cache_pages_needed(void* c, int64_t rid, int from_len, int new_len, int g) {
  return static_cast<CacheManager*>(c)->pages_needed(rid, from_len, new_len, g);
}
int dn_cache_pages_peak(void* c, int g, int total_len, int chunk) {
  return static_cast<CacheManager*>(c)->pages_peak(g, total_len, chunk);
}
int dn_cache_lengths(void* c, const int64_t* rids, int n, int* out, int* failed) {
  return static_cast<CacheManager*>(c)->lengths(rids, n, out, failed);
}
int dn_cache_reserve_step(void* c, const int64_t* rids, const int* new_lens, int n, int* slots_out, int* failed) {
  return static_cast<CacheManager*>(c)->reserve_step(rids, new_lens, n, slots_out, failed);
}
int dn_cache_commit_step(void* c, const int64_t* rids, const int* new_lens, int n, int* failed) {
  return static_cast<CacheManager*>(c)->commit_step(rids, new_lens, n, failed);
}
int dn_cache_max_blocks(void* c, int g, const int64_t* rids, int n) {
  return static_cast<CacheManager*>(c)->max_blocks(g, rids, n);
}
int dn_cache_step_tables(void* c, int g, const int64_t* rids, const int* starts, const int* counts, int n,
                         int bt_rows, int max_blocks, int32_t* block_tables, int32_t* slot_map, int sm_len,
                         int* failed) {
  return static_cast<CacheManager*>(c)->step_tables(g, rids, starts, counts, n, bt_rows, max_blocks, block_tables,
                                                    slot_map, sm_len, failed);
}
int dn_cache_live(void* c) { return static_cast<CacheManager*>(c)->live(); }
int dn_cache_check(void* c) { return static_cast<CacheManager*>(c)->check(); }
int64_t dn_cache_reuse_count(void* c, int g) { return static_cast<CacheManager*>(c)->reuse_count(g); }

void* dn_sched_create(void* cache, int max_live, int max_batch_tokens, int prefill_chunk, int policy,
                      int max_positions) {
  if (!cache || max_live < 1 || max_batch_tokens < 1 || prefill_chunk < 1 || max_positions < 1) return nullptr;
  return new (std::nothrow) Scheduler(static_cast<CacheManager*>(cache), max_live, max_batch_tokens,
                                      prefill_chunk, policy, max_positions);
}
void dn_sched_destroy(void* s) { delete static_cast<Scheduler*>(s); }
int dn_sched_add(void* s, int64_t rid, int prompt_len, int max_new) {
  return static_cast<Scheduler*>(s)->add(rid, prompt_len, max_new);
}
// entries: rid[i], start[i], count[i], samples[i]; returns the number of entries, or -1 if cap is too small
int dn_sched_schedule(void* s, int64_t* rid, int* start, int* count, int* samples, int cap,
                      int64_t* preempted, int* n_preempted, int cap_preempted) {
  std::vector<StepEntry> out;
  std::vector<int64_t> pre;
  static_cast<Scheduler*>(s)->schedule(&out, &pre);
  if (static_cast<int>(out.size()) > cap || static_cast<int>(pre.size()) > cap_preempted) return -1;
  for (size_t i = 0; i < out.size(); ++i) {
    rid[i] = out[i].rid;
    start[i] = out[i].start;
    count[i] = out[i].count;
    samples[i] = out[i].samples;
  }
  for (size_t i = 0; i < pre.size(); ++i) preempted[i] = pre[i];
  *n_preempted = static_cast<int>(pre.size());
  return static_cast<int>(out.size());
}
int dn_sched_step_done(void* s, int64_t rid, int count) { return static_cast<Scheduler*>(s)->step_done(rid, count); }
int dn_sched_token_sampled(void* s, int64_t rid) { return static_cast<Scheduler*>(s)->token_sampled(rid); }
int dn_sched_steps_done(void* s, const int64_t* rids, const int* counts, int n, int* failed) {
  return static_cast<Scheduler*>(s)->steps_done(rids, counts, n, failed);
}
int dn_sched_tokens_sampled(void* s, const int64_t* rids, int n, int* last, int* failed) {
  return static_cast<Scheduler*>(s)->tokens_sampled(rids, n, last, failed);
}
int dn_sched_finish(void* s, int64_t rid) { return static_cast<Scheduler*>(s)->finish(rid); }
int dn_sched_n_waiting(void* s) { return static_cast<Scheduler*>(s)->n_waiting(); }
int dn_sched_n_running(void* s) { return static_cast<Scheduler*>(s)->n_running(); }
int dn_sched_known(void* s, int64_t rid) { return static_cast<Scheduler*>(s)->known(rid); }
int dn_sched_computed(void* s, int64_t rid) { return static_cast<Scheduler*>(s)->computed(rid); }
int dn_sched_generated(void* s, int64_t rid) { return static_cast<Scheduler*>(s)->generated(rid); }

}  // extern "C"
