#include "scheduler.h"

#include <algorithm>

namespace xi {

Scheduler::Scheduler(CacheManager* cm, int max_num_seqs, int max_batched_tokens, int chunk_size)
    : cm_(cm),
      max_num_seqs_(std::max(1, max_num_seqs)),
      max_batched_tokens_(std::max(1, max_batched_tokens)),
      chunk_size_(std::max(1, chunk_size)) {}

const SchedRequest* Scheduler::find(int64_t id) const {
  auto it = requests_.find(id);
  return it == requests_.end() ? nullptr : &it->second;
}

int Scheduler::add(int64_t id, int64_t prompt_len, int64_t max_new_tokens) {
  if (prompt_len <= 0 || max_new_tokens < 0) {
    error_ = "a request needs at least one prompt token";
    return -3;
  }
  if (requests_.count(id) || cm_->has(id)) {
    error_ = "request " + std::to_string(id) + " exists already";
    return -2;
  }
  const int64_t max_len = prompt_len + max_new_tokens;
  for (int g = 0; g < cm_->num_groups(); ++g) {
    const GroupSpec& grp = cm_->group(g);
    // A group that keeps every key holds the whole request at its end.  A group with a window
    // holds, while a portion of n tokens runs, the window - 1 keys before it and its own n: one
    // page more than those tokens fill, since they need not start at a page's edge.
    int64_t held = max_len;
    int64_t pages = (max_len + grp.page_size - 1) / grp.page_size;
    if (grp.window > 0) {
      const int64_t portion = std::min<int64_t>(chunk_size_, max_batched_tokens_);
      held = std::min<int64_t>(max_len, (int64_t)grp.window - 1 + portion);
      pages = std::min<int64_t>(pages, (held + grp.page_size - 1) / grp.page_size + 1);
    }
    if (pages > grp.num_pages) {
      error_ = "request of " + std::to_string(prompt_len) + " prompt tokens and up to " +
               std::to_string(max_new_tokens) + " new tokens needs " + std::to_string(pages) +
               " cache pages but the pool has " + std::to_string(grp.num_pages);
      return -1;
    }
  }
  SchedRequest r;
  r.id = id;
  r.prompt_len = r.total_len = prompt_len;
  r.max_len = max_len;
  requests_.emplace(id, r);
  waiting_.push_back(id);
  return 0;
}

void Scheduler::preempt(int64_t id) {
  SchedRequest& r = requests_.at(id);
  cm_->release(id);
  r.computed = 0;
  r.running = false;
  running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
  plan_.erase(std::remove_if(plan_.begin(), plan_.end(), [&](const SchedEntry& e) { return e.id == id; }),
              plan_.end());
  waiting_.push_front(id);
}

const std::vector<SchedEntry>& Scheduler::schedule(std::vector<int64_t>* preempted) {
  plan_.clear();
  int64_t budget = max_batched_tokens_;
  bool preempted_any = false;

  // 1 and 2: running requests, oldest first; decoding ones first, then unfinished prompts.
  for (int pass = 0; pass < 2; ++pass) {
    const std::vector<int64_t> order = running_;
    for (int64_t id : order) {
      auto it = requests_.find(id);
      if (it == requests_.end() || !it->second.running) continue;  // preempted meanwhile
      SchedRequest& r = it->second;
      const int64_t remaining = r.total_len - r.computed;
      const bool decoding = remaining == 1 && r.computed >= r.prompt_len;
      if ((pass == 0) != decoding) continue;
      if (remaining <= 0 || budget <= 0) continue;
      const int64_t n = std::min<int64_t>({remaining, (int64_t)chunk_size_, budget});
      bool ok = true;
      while (!cm_->reserve(id, n)) {
        // out of pages: the youngest running request gives way
        int64_t victim = running_.back();
        int64_t best = -1;
        for (int64_t cand : running_)
          if (requests_.at(cand).order > best) { best = requests_.at(cand).order; victim = cand; }
        budget += [&] { int64_t s = 0; for (auto& e : plan_) if (e.id == victim) s += e.count; return s; }();
        preempt(victim);
        preempted_any = true;
        if (preempted) preempted->push_back(victim);
        if (victim == id) { ok = false; break; }
      }
      if (!ok) continue;
      plan_.push_back(SchedEntry{id, r.computed, (int32_t)n, r.computed + n == r.total_len ? 1 : 0});
      budget -= n;
    }
  }

  // 3: admissions, in queue order, while everything allows.  A new request gets pages for
  // all of its known tokens at once (as the reference allocates a whole prompt,
  // block_manager.rs:132-147), so its later portions cannot run out of pages, in the groups that
  // keep every key; in a group with a window it gets the first portion's pages, and each later
  // portion takes its own after the pages behind the window have gone back (if the pool is
  // short then, the youngest request gives way as for any other growth).
  // Nothing is admitted in a step that had to preempt: pages are short.
  while (!preempted_any && !waiting_.empty() && budget > 0 && (int)running_.size() < max_num_seqs_ &&
         cm_->free_state_slots() > 0) {
    const int64_t id = waiting_.front();
    SchedRequest& r = requests_.at(id);
    if (cm_->add_request(id) < 0) break;
    const int64_t n = std::min<int64_t>({r.total_len, (int64_t)chunk_size_, budget});
    if (!cm_->reserve(id, n, r.total_len)) {
      cm_->release(id);
      break;
    }
    waiting_.pop_front();
    r.running = true;
    r.order = next_order_++;
    running_.push_back(id);
    plan_.push_back(SchedEntry{id, 0, (int32_t)n, n == r.total_len ? 1 : 0});
    budget -= n;
  }

  // The decoding requests at the head of the step, longest first: the attention kernel's workgroups
  // start in the batch's order, and the long sequences' then do not run on alone at the end.
  size_t decoding = 0;
  while (decoding < plan_.size()) {
    const SchedEntry& e = plan_[decoding];
    const SchedRequest& r = requests_.at(e.id);
    if (e.count != 1 || e.start < r.prompt_len || e.start + 1 != r.total_len) break;
    ++decoding;
  }
  std::stable_sort(plan_.begin(), plan_.begin() + decoding,
                   [](const SchedEntry& a, const SchedEntry& b) { return a.start > b.start; });
  return plan_;
}

void Scheduler::commit() {
  for (const SchedEntry& e : plan_) {
    auto it = requests_.find(e.id);
    if (it == requests_.end() || !it->second.running) continue;
    if (cm_->commit(e.id, e.count) < 0) {
      error_ = cm_->last_error();
      continue;
    }
    it->second.computed += e.count;
  }
  plan_.clear();
}

int Scheduler::append_token(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return -1;
  if (it->second.total_len >= it->second.max_len) return -1;
  it->second.total_len += 1;
  return 0;
}

int Scheduler::finish(int64_t id) {
  auto it = requests_.find(id);
  if (it == requests_.end()) return -1;
  if (it->second.running) {
    cm_->release(id);
    running_.erase(std::remove(running_.begin(), running_.end(), id), running_.end());
  } else {
    waiting_.erase(std::remove(waiting_.begin(), waiting_.end(), id), waiting_.end());
  }
  plan_.erase(std::remove_if(plan_.begin(), plan_.end(), [&](const SchedEntry& e) { return e.id == id; }),
              plan_.end());
  requests_.erase(it);
  return 0;
}

}  // namespace xi
