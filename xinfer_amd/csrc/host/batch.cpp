// Turns a step's entries (request, number of new tokens) into the flat arrays the
// kernels read.  The reference builds the same set in prepare_prefill / prepare_decode
// (/root/reference/src/core/runner.rs:1303-1563, 1565-1750); here one builder serves both,
// a decode token being a portion of one token.
#include <cstring>

#include "cache.h"

using xi::CacheManager;
using xi::RequestPages;

extern "C" {

// The longest block table among the given requests, over all groups (at least 1).
int xi_cm_max_table_len(CacheManager* cm, int B, const int64_t* ids) {
  size_t longest = 1;
  for (int b = 0; b < B; ++b) {
    const RequestPages* r = cm->find(ids[b]);
    if (!r) return -1;
    for (const auto& t : r->tables) longest = t.size() > longest ? t.size() : longest;
  }
  return (int)longest;
}

// Fills, for B entries with T tokens in total:
//   positions[T], tok_seq[T], cu_q[B+1], ctx_lens[B], state_slots[B]
//   slots[G][T]                     cache slot of each new token per group
//   block_tables[G][B][max_pages]   physical pages, 0 where none is held
// Pages must have been reserved.  Returns 0, or a negative code with the manager's
// last_error set.
int xi_cm_build_batch(CacheManager* cm, int B, const int64_t* ids, const int32_t* n_tokens,
                      int32_t* positions, int32_t* tok_seq, int32_t* cu_q, int32_t* ctx_lens,
                      int32_t* state_slots, int64_t* slots, int32_t* block_tables,
                      int max_pages, int T) {
  const int G = cm->num_groups();
  int t = 0;
  cu_q[0] = 0;
  for (int b = 0; b < B; ++b) {
    const RequestPages* r = cm->find(ids[b]);
    if (!r) return -1;
    const int n = n_tokens[b];
    if (n <= 0 || t + n > T) return -2;
    if (r->length + n > r->reserved) return -3;
    for (int i = 0; i < n; ++i) {
      positions[t + i] = (int32_t)(r->length + i);
      tok_seq[t + i] = b;
    }
    for (int g = 0; g < G; ++g) {
      const auto& table = r->tables[g];
      if ((int)table.size() > max_pages) return -4;
      int32_t* bt = block_tables + ((size_t)g * B + b) * max_pages;
      for (int p = 0; p < max_pages; ++p)
        bt[p] = (p < (int)table.size() && table[p] >= 0) ? table[p] : 0;
      for (int i = 0; i < n; ++i) {
        const int64_t s = cm->slot_of(*r, g, r->length + i);
        if (s < 0) return -5;
        slots[(size_t)g * T + t + i] = s;
      }
    }
    ctx_lens[b] = (int32_t)(r->length + n);
    state_slots[b] = r->state_slot;
    t += n;
    cu_q[b + 1] = t;
  }
  return t == T ? 0 : -6;
}

}  // extern "C"
