// Continuous-batching scheduler.
//
// Every step fills a token budget with, in this order: one token for each running request
// that is decoding; the next portion of each running request whose prompt is not yet in
// the cache; portions of newly admitted requests while the budget, the number of live
// requests and the pages allow.  Portions and decode tokens share one batch.
//
// The reference alternates prefill-only and decode-only steps and re-queues unfinished
// prompts (/root/reference/src/core/scheduler.rs:236-408, 821-899); its chunk arithmetic
// is Sequence::prefill_chunk_tokens (/root/reference/src/core/sequence.rs:223-243).
//
// When pages run out while running requests grow, the youngest running request is
// preempted: its pages are given back and it returns to the head of the waiting queue,
// to be recomputed from its first token (prompt and generated tokens alike) when pages
// are free again.  The reference instead skips, swaps to host memory or cancels
// (scheduler.rs:346-387, engine.rs:1604-1621).  A request that could never fit, even
// alone, is refused when it is added (reference: engine.rs:730-776).
#pragma once
#include <cstdint>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

#include "cache.h"

namespace xi {

struct SchedRequest {
  int64_t id = 0;
  int64_t total_len = 0;    // known tokens: prompt and generated
  int64_t prompt_len = 0;
  int64_t max_len = 0;      // prompt + most tokens it may generate
  int64_t computed = 0;     // tokens in the cache
  int64_t order = 0;        // admission order (larger = younger)
  bool running = false;
};

struct SchedEntry {
  int64_t id;
  int64_t start;   // position of the entry's first token
  int32_t count;   // number of tokens
  int32_t sample;  // 1 if the entry ends at the request's last known token
};

class Scheduler {
 public:
  Scheduler(CacheManager* cm, int max_num_seqs, int max_batched_tokens, int chunk_size);

  // 0 ok; -1 the request can never fit in the cache; -2 duplicate id; -3 bad sizes.
  int add(int64_t id, int64_t prompt_len, int64_t max_new_tokens);
  // Plans one step and reserves its pages.  Ids preempted while planning are appended to
  // `preempted`.
  const std::vector<SchedEntry>& schedule(std::vector<int64_t>* preempted);
  // The planned step ran: its tokens are in the cache (recorded in the cache manager too).
  void commit();
  // A sampled token joins the request's known tokens.  -1 if unknown or beyond max_len.
  int append_token(int64_t id);
  // The request is done (or cancelled): give back what it holds.  -1 if unknown.
  int finish(int64_t id);

  int num_waiting() const { return (int)waiting_.size(); }
  int num_running() const { return (int)running_.size(); }
  const SchedRequest* find(int64_t id) const;
  const std::string& last_error() const { return error_; }

 private:
  void preempt(int64_t id);

  CacheManager* cm_;
  int max_num_seqs_, max_batched_tokens_, chunk_size_;
  int64_t next_order_ = 0;
  std::unordered_map<int64_t, SchedRequest> requests_;
  std::deque<int64_t> waiting_;
  std::vector<int64_t> running_;  // in admission order
  std::vector<SchedEntry> plan_;
  std::string error_;
};

}  // namespace xi
