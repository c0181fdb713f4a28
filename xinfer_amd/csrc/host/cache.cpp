#include "cache.h"

#include <algorithm>

namespace xi {

CacheManager::CacheManager(const std::vector<GroupSpec>& groups, int max_requests)
    : groups_(groups) {
  free_.resize(groups_.size());
  held_.resize(groups_.size());
  for (size_t g = 0; g < groups_.size(); ++g) {
    for (int p = 0; p < groups_[g].num_pages; ++p) free_[g].push_back(p);
    held_[g].assign((size_t)std::max(groups_[g].num_pages, 0), 0);
  }
  for (int s = max_requests - 1; s >= 0; --s) free_slots_.push_back(s);  // lowest slot first
}

const RequestPages* CacheManager::find(int64_t id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? nullptr : &it->second;
}

int CacheManager::add_request(int64_t id) {
  if (requests_.count(id)) return -2;
  if (free_slots_.empty()) return -1;
  RequestPages r;
  r.state_slot = free_slots_.back();
  free_slots_.pop_back();
  r.tables.resize(groups_.size());
  r.first_held.assign(groups_.size(), 0);
  const int slot = r.state_slot;
  requests_.emplace(id, std::move(r));
  return slot;
}

static inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

int CacheManager::pages_needed(int64_t id, int64_t n, int g) const {
  const RequestPages* r = find(id);
  if (!r || n < 0) return -1;
  const int64_t want = ceil_div(r->length + n, groups_[g].page_size);
  const int64_t have = (int64_t)r->tables[g].size();
  return (int)std::max<int64_t>(0, want - have);
}

// Tokens for which group g takes pages when n run next and `ahead` are known to follow.
static inline int64_t tokens_of(const GroupSpec& grp, int64_t n, int64_t ahead) {
  return grp.window > 0 ? n : std::max(n, ahead);
}

bool CacheManager::can_reserve(int64_t id, int64_t n, int64_t ahead) const {
  if (!find(id) || n < 0) return false;
  for (int g = 0; g < num_groups(); ++g)
    if (pages_needed(id, tokens_of(groups_[g], n, ahead), g) > free_pages(g)) return false;
  return true;
}

bool CacheManager::reserve(int64_t id, int64_t n, int64_t ahead) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "reserve: unknown request " + std::to_string(id);
    return false;
  }
  if (!can_reserve(id, n, ahead)) {
    error_ = "No free blocks available, retry later!";  // block_manager.rs:139
    return false;
  }
  RequestPages& r = it->second;
  for (int g = 0; g < num_groups(); ++g) {
    const int need = pages_needed(id, tokens_of(groups_[g], n, ahead), g);
    for (int i = 0; i < need; ++i) {
      const int32_t p = free_[g].front();
      free_[g].pop_front();
      held_[g][p] = 1;
      r.tables[g].push_back(p);
    }
  }
  r.reserved = std::max(r.reserved, r.length + n);
  return true;
}

int CacheManager::commit(int64_t id, int64_t n) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "commit: unknown request " + std::to_string(id);
    return -1;
  }
  RequestPages& r = it->second;
  if (n < 0 || r.length + n > r.reserved) {
    error_ = "commit: request " + std::to_string(id) + " has pages for " +
             std::to_string(r.reserved) + " tokens, cannot hold " + std::to_string(r.length + n);
    return -1;
  }
  r.length += n;
  int given_back = 0;
  for (int g = 0; g < num_groups(); ++g) {
    const int w = groups_[g].window;
    if (w <= 0) continue;
    // the next query sits at position `length`; it and all later ones see keys >= length-w+1
    const int64_t first_key = r.length - w + 1;
    if (first_key <= 0) continue;
    const int64_t first_page = std::min<int64_t>(first_key / groups_[g].page_size,
                                                 (int64_t)r.tables[g].size());
    for (int64_t p = r.first_held[g]; p < first_page; ++p) {
      const int32_t phys = r.tables[g][p];
      if (phys < 0) continue;
      held_[g][phys] = 0;
      free_[g].push_back(phys);
      r.tables[g][p] = -1;
      ++given_back;
    }
    r.first_held[g] = std::max(r.first_held[g], first_page);
  }
  return given_back;
}

int CacheManager::release(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) {
    error_ = "release: unknown request " + std::to_string(id);
    return -1;
  }
  RequestPages& r = it->second;
  int n = 0;
  for (int g = 0; g < num_groups(); ++g) {
    for (int32_t phys : r.tables[g]) {
      if (phys < 0) continue;
      held_[g][phys] = 0;
      free_[g].push_back(phys);
      ++n;
    }
  }
  free_slots_.push_back(r.state_slot);
  requests_.erase(it);
  return n;
}

int64_t CacheManager::slot_of(const RequestPages& r, int g, int64_t pos) const {
  const int ps = groups_[g].page_size;
  const int64_t lp = pos / ps;
  if (lp < 0 || lp >= (int64_t)r.tables[g].size()) return -1;
  const int32_t phys = r.tables[g][lp];
  if (phys < 0) return -1;
  return (int64_t)phys * ps + pos % ps;
}

bool CacheManager::check_invariants(std::string* why) const {
  for (int g = 0; g < num_groups(); ++g) {
    std::vector<int> seen((size_t)groups_[g].num_pages, 0);
    for (int32_t p : free_[g]) {
      if (p < 0 || p >= groups_[g].num_pages) { if (why) *why = "free list holds a bad page id"; return false; }
      if (seen[p]++) { if (why) *why = "page " + std::to_string(p) + " is free twice"; return false; }
      if (held_[g][p]) { if (why) *why = "page " + std::to_string(p) + " is free and held"; return false; }
    }
    for (const auto& kv : requests_) {
      for (int32_t p : kv.second.tables[g]) {
        if (p < 0) continue;
        if (p >= groups_[g].num_pages) { if (why) *why = "table holds a bad page id"; return false; }
        if (seen[p]++) { if (why) *why = "page " + std::to_string(p) + " is held twice or also free"; return false; }
        if (!held_[g][p]) { if (why) *why = "page " + std::to_string(p) + " is in a table but not marked held"; return false; }
      }
    }
    for (int p = 0; p < groups_[g].num_pages; ++p)
      if (!seen[p]) { if (why) *why = "page " + std::to_string(p) + " of group " + std::to_string(g) + " is lost"; return false; }
  }
  std::vector<int> slot_seen(free_slots_.size() + requests_.size(), 0);
  for (int s : free_slots_) {
    if (s < 0 || s >= (int)slot_seen.size() || slot_seen[s]++) { if (why) *why = "state slot free twice"; return false; }
  }
  for (const auto& kv : requests_) {
    const int s = kv.second.state_slot;
    if (s < 0 || s >= (int)slot_seen.size() || slot_seen[s]++) { if (why) *why = "state slot held twice"; return false; }
  }
  return true;
}

}  // namespace xi
