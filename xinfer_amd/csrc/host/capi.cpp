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

}  // extern "C"
