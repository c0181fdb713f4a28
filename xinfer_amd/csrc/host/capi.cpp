// C interface of the host runtime, loaded from Python with ctypes.
#include <cstring>
#include <string>

#include "cache.h"

using xi::CacheManager;
using xi::GroupSpec;

extern "C" {

CacheManager* xi_cm_create(int num_groups, const int32_t* page_sizes, const int32_t* num_pages,
                           const int32_t* windows, int max_requests) {
  if (num_groups <= 0 || max_requests <= 0) return nullptr;
  std::vector<GroupSpec> g((size_t)num_groups);
  for (int i = 0; i < num_groups; ++i) {
    if (page_sizes[i] <= 0 || num_pages[i] < 0 || windows[i] < 0) return nullptr;
    g[i] = GroupSpec{page_sizes[i], num_pages[i], windows[i]};
  }
  return new CacheManager(g, max_requests);
}
void xi_cm_destroy(CacheManager* cm) { delete cm; }

int xi_cm_num_groups(CacheManager* cm) { return cm->num_groups(); }
int xi_cm_free_pages(CacheManager* cm, int g) { return cm->free_pages(g); }
int xi_cm_free_state_slots(CacheManager* cm) { return cm->free_state_slots(); }
int xi_cm_live_requests(CacheManager* cm) { return cm->live_requests(); }
int xi_cm_has(CacheManager* cm, int64_t id) { return cm->has(id) ? 1 : 0; }
int xi_cm_add_request(CacheManager* cm, int64_t id) { return cm->add_request(id); }
int xi_cm_pages_needed(CacheManager* cm, int64_t id, int64_t n, int g) { return cm->pages_needed(id, n, g); }
int xi_cm_can_reserve(CacheManager* cm, int64_t id, int64_t n) { return cm->can_reserve(id, n) ? 1 : 0; }
int xi_cm_reserve(CacheManager* cm, int64_t id, int64_t n) { return cm->reserve(id, n) ? 1 : 0; }
int xi_cm_commit(CacheManager* cm, int64_t id, int64_t n) { return cm->commit(id, n); }
int xi_cm_release(CacheManager* cm, int64_t id) { return cm->release(id); }
int64_t xi_cm_length(CacheManager* cm, int64_t id) {
  const xi::RequestPages* r = cm->find(id);
  return r ? r->length : -1;
}
int xi_cm_state_slot(CacheManager* cm, int64_t id) {
  const xi::RequestPages* r = cm->find(id);
  return r ? r->state_slot : -1;
}
// Copies the block table of (id, group) into out (at most cap entries); returns its length.
int xi_cm_block_table(CacheManager* cm, int64_t id, int g, int32_t* out, int cap) {
  const xi::RequestPages* r = cm->find(id);
  if (!r || g < 0 || g >= cm->num_groups()) return -1;
  const auto& t = r->tables[g];
  for (int i = 0; i < (int)t.size() && i < cap; ++i) out[i] = t[i];
  return (int)t.size();
}
int xi_cm_check(CacheManager* cm, char* why, int cap) {
  std::string w;
  const bool ok = cm->check_invariants(&w);
  if (why && cap > 0) {
    std::strncpy(why, w.c_str(), (size_t)cap - 1);
    why[cap - 1] = 0;
  }
  return ok ? 1 : 0;
}
const char* xi_cm_last_error(CacheManager* cm) { return cm->last_error().c_str(); }

// The same for many requests in one call (a step's worth): lengths (-1: not live); reserve until
// one fails (returns its index, or -1 if all succeeded); commit all (returns 0, or -1 - index of
// the first that failed, the ones before it committed).
void xi_cm_lengths(CacheManager* cm, int B, const int64_t* ids, int64_t* out) {
  for (int b = 0; b < B; ++b) {
    const xi::RequestPages* r = cm->find(ids[b]);
    out[b] = r ? r->length : -1;
  }
}
int xi_cm_reserve_many(CacheManager* cm, int B, const int64_t* ids, const int32_t* counts) {
  for (int b = 0; b < B; ++b)
    if (!cm->reserve(ids[b], counts[b])) return b;
  return -1;
}
int xi_cm_commit_many(CacheManager* cm, int B, const int64_t* ids, const int32_t* counts) {
  for (int b = 0; b < B; ++b)
    if (cm->commit(ids[b], counts[b]) < 0) return -1 - b;
  return 0;
}

}  // extern "C"

// ---- scheduler -----------------------------------------------------------------------
#include "scheduler.h"

using xi::Scheduler;

extern "C" {

Scheduler* xi_sched_create(CacheManager* cm, int max_num_seqs, int max_batched_tokens, int chunk_size) {
  return cm ? new Scheduler(cm, max_num_seqs, max_batched_tokens, chunk_size) : nullptr;
}
void xi_sched_destroy(Scheduler* s) { delete s; }
int xi_sched_add(Scheduler* s, int64_t id, int64_t prompt_len, int64_t max_new_tokens) {
  return s->add(id, prompt_len, max_new_tokens);
}
// Plans a step.  Writes up to cap entries and up to pre_cap preempted ids; returns the
// number of entries (or -1 if cap is too small), *n_preempted the number of preempted.
int xi_sched_schedule(Scheduler* s, int64_t* ids, int64_t* starts, int32_t* counts, int32_t* sample,
                      int cap, int64_t* preempted, int pre_cap, int32_t* n_preempted) {
  std::vector<int64_t> pre;
  const auto& plan = s->schedule(&pre);
  *n_preempted = (int32_t)pre.size();
  for (int i = 0; i < (int)pre.size() && i < pre_cap; ++i) preempted[i] = pre[i];
  if ((int)plan.size() > cap) return -1;
  for (size_t i = 0; i < plan.size(); ++i) {
    ids[i] = plan[i].id;
    starts[i] = plan[i].start;
    counts[i] = plan[i].count;
    sample[i] = plan[i].sample;
  }
  return (int)plan.size();
}
void xi_sched_commit(Scheduler* s) { s->commit(); }
int xi_sched_append_token(Scheduler* s, int64_t id) { return s->append_token(id); }
int xi_sched_finish(Scheduler* s, int64_t id) { return s->finish(id); }
int xi_sched_num_waiting(Scheduler* s) { return s->num_waiting(); }
int xi_sched_num_running(Scheduler* s) { return s->num_running(); }
int64_t xi_sched_computed(Scheduler* s, int64_t id) {
  const xi::SchedRequest* r = s->find(id);
  return r ? r->computed : -1;
}
const char* xi_sched_last_error(Scheduler* s) { return s->last_error().c_str(); }

}  // extern "C"
