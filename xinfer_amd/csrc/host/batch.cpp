// Turns a step's entries (request, number of new tokens) into the flat arrays the
// kernels read.  The reference builds the same set in prepare_prefill / prepare_decode
// (/root/reference/src/core/runner.rs:1303-1563, 1565-1750); here one builder serves both,
// a decode token being a portion of one token.
#include <cstring>
#include <vector>

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

// A step in which every one of B requests brings one token, prepared in one call for the
// recorded (graph) path: checks the requests (live, once each, within max_positions, token in
// the vocabulary), reserves one token each if `reserve`, and writes the step's arrays in the
// layout of the runner's two upload buffers:
//   out32 = ids[B] positions[B] tok_seq[B] cu_q[B+1] ctx_lens[B] rows[B] block_tables[G][B][max_pages]
//   out64 = state_slots[B] slots[G][B] no_slots[B] (= -1)
// rows: the n_rows wanted rows first, zeros after.  stats[0] = the longest cached length after
// the step, stats[1] = 1 if the mean length is at least 0.9 of the longest.
// Returns 0, or a negative kind with *bad = the entry: -1 not live, -2 twice, -3 past
// max_positions, -4 token outside the vocabulary, -5 no pages (entries before it keep theirs),
// -6 a wanted row outside the step, -7 the batch could not be built (last_error says why).
int xi_cm_decode_step(CacheManager* cm, int B, const int64_t* ids, const int32_t* tokens, int reserve, int vocab,
                      int64_t max_positions, int max_pages, const int32_t* rows, int n_rows, int32_t* out32,
                      int64_t* out64, int32_t* stats, int32_t* bad) {
  const int G = cm->num_groups();
  for (int b = 0; b < B; ++b) {
    *bad = b;
    const RequestPages* r = cm->find(ids[b]);
    if (!r) return -1;
    for (int a = 0; a < b; ++a)
      if (ids[a] == ids[b]) return -2;
    if (r->length + 1 > max_positions) return -3;
    if (tokens[b] < 0 || tokens[b] >= vocab) return -4;
  }
  for (int i = 0; i < n_rows; ++i) {
    *bad = i;
    if (rows[i] < 0 || rows[i] >= B) return -6;
  }
  if (reserve)
    for (int b = 0; b < B; ++b) {
      *bad = b;
      if (!cm->reserve(ids[b], 1)) return -5;
    }
  int32_t* o_ids = out32;
  int32_t* o_pos = o_ids + B;
  int32_t* o_seq = o_pos + B;
  int32_t* o_cu = o_seq + B;
  int32_t* o_ctx = o_cu + B + 1;
  int32_t* o_rows = o_ctx + B;
  int32_t* o_bt = o_rows + B;
  int64_t* o_state = out64;
  int64_t* o_slots = o_state + B;
  int64_t* o_none = o_slots + (size_t)G * B;
  std::vector<int32_t> ones((size_t)B, 1), state32((size_t)B);
  const int rc = xi_cm_build_batch(cm, B, ids, ones.data(), o_pos, o_seq, o_cu, o_ctx, state32.data(), o_slots, o_bt,
                                   max_pages, B);
  if (rc != 0) {
    *bad = rc;
    return -7;
  }
  int64_t longest = 0, total = 0;
  for (int b = 0; b < B; ++b) {
    o_ids[b] = tokens[b];
    o_rows[b] = b < n_rows ? rows[b] : 0;
    o_state[b] = state32[(size_t)b];
    o_none[b] = -1;
    longest = o_ctx[b] > longest ? o_ctx[b] : longest;
    total += o_ctx[b];
  }
  stats[0] = (int32_t)longest;
  stats[1] = ((double)total / B >= 0.9 * (double)longest) ? 1 : 0;
  return 0;
}

}  // extern "C"
