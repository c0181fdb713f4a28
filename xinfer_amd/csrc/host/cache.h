// Paged cache bookkeeping on the host: which request holds which pages.
//
// Layers with the same needs form a group; every group has a page pool of its own and
// every request has one block table per group.  A group either keeps all keys
// (window == 0) or only the last `window` of them, in which case pages that every
// later query's window has passed are given back while the request is still running.
// Beside the pages each live request owns one slot of fixed-size state.
//
// The reference's counterpart is BlockManager (/root/reference/src/core/block_manager.rs:
// 19-56 blocks and FIFO free list, 124-161 allocate, 273-320 append with rollback,
// 331-337 deallocate) and the MambaCache slots (/root/reference/src/core/runner.rs:252-289).
#pragma once
#include <cstdint>
#include <deque>
#include <string>
#include <unordered_map>
#include <vector>

namespace xi {

struct GroupSpec {
  int page_size;
  int num_pages;
  int window;  // 0: every key is kept
};

struct RequestPages {
  int64_t length = 0;    // tokens whose keys and values are in the cache
  int64_t reserved = 0;  // tokens for which pages are reserved (>= length)
  int state_slot = -1;
  std::vector<std::vector<int32_t>> tables;  // [group][logical page] -> physical page or -1
  std::vector<int64_t> first_held;           // [group] first logical page still held
};

class CacheManager {
 public:
  CacheManager(const std::vector<GroupSpec>& groups, int max_requests);

  int num_groups() const { return (int)groups_.size(); }
  const GroupSpec& group(int g) const { return groups_[g]; }
  int free_pages(int g) const { return (int)free_[g].size(); }
  int free_state_slots() const { return (int)free_slots_.size(); }
  int live_requests() const { return (int)requests_.size(); }
  bool has(int64_t id) const { return requests_.count(id) != 0; }
  const RequestPages* find(int64_t id) const;

  // Returns the state slot (>= 0), -1 if no slot is free, -2 if the id is live already.
  int add_request(int64_t id);
  // Pages that `reserve(id, n)` would have to take from group g's pool.
  int pages_needed(int64_t id, int64_t n, int g) const;
  bool can_reserve(int64_t id, int64_t n, int64_t ahead = 0) const;
  // Reserves pages for the next n tokens of the request in every group, or changes
  // nothing and returns false when a pool has too few free pages.  `ahead` > n: groups that
  // keep every key reserve for that many tokens at once (a prompt admitted whole, of which n
  // tokens run first); a group with a window takes pages for the n tokens alone, since by the
  // time the later ones run it has given earlier pages back.
  bool reserve(int64_t id, int64_t n, int64_t ahead = 0);
  // The next n tokens are now in the cache.  Gives back window pages no later query needs.
  // Returns the number of pages given back, or -1 on misuse (see last_error()).
  int commit(int64_t id, int64_t n);
  // Gives back everything the request holds.  Returns the number of pages, -1 if unknown.
  int release(int64_t id);

  // Slot of token position `pos` of a request in group g: page * page_size + offset.
  int64_t slot_of(const RequestPages& r, int g, int64_t pos) const;

  // Consistency: every page is either free or held by exactly one live table, once.
  bool check_invariants(std::string* why) const;

  const std::string& last_error() const { return error_; }

 private:
  std::vector<GroupSpec> groups_;
  std::vector<std::deque<int32_t>> free_;  // FIFO: taken from the front, returned to the back
  std::vector<std::vector<uint8_t>> held_; // [group][page] 1 while a request holds it
  std::vector<int> free_slots_;
  std::unordered_map<int64_t, RequestPages> requests_;
  mutable std::string error_;
};

}  // namespace xi
