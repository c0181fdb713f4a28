// bfloat16 paged causal GQA attention on the gfx950 matrix cores: the wave-level step and
// the split-K decode kernels (the prefill kernel, attention_prefill.hip, stages the same
// operands through LDS).
//
// The wave-level step: 32 keys against NQT tiles of 16 query
// columns, with v_mfma_f32_16x16x32_bf16 and no transposes through LDS:
//
//   S^T[key, q] = K[key, :] . Q[q, :]          A = K rows      B = Q^T
//   O^T[d, q]  += V^T[d, key] * P^T[key, q]    A = V^T rows    B = P^T
//
// A-operand lane l holds row l%16 and 8 contiguous elements of the contraction index
// (group l/16); B-operand lane l holds column l%16 and the same 8 elements; the 16x16
// result has lane l holding column l%16, rows 4*(l/16)..+3.  So a lane's S^T results are
// 4 consecutive keys of its own query column, which is exactly a B operand of the second
// product once rounded to bfloat16 - provided the V^T operand pairs the same keys with the
// same slots.  Row m of the two K tiles of a step is therefore key 8*(m/4) + m%4 (tile 0)
// and that + 4 (tile 1): lane group j then holds keys 8j..8j+7, one 16-byte load from V^T.
//
// The cache keeps K as [page, kv_head, offset, d] and V in groups of eight keys as
// [page, kv_head, offset / 8, d, 8], so both operands are read from global memory in the layout
// the matrix cores want: a lane's 16 bytes of V^T are eight keys of one dim, sixteen dims lie side
// by side (a wave's load of a step takes four runs of 256 bytes a tile; with a whole page's keys
// side by side it took sixteen half lines, and a new token's value d lines of the pool instead of
// d / 8: 64 sequences of 4,096 keys went from 190 to 178 us, 256 of 1,024 from 233 to 202).  Softmax runs in float32 (exp2 with log2(e) folded into the
// scale); all per-query state (running max, sum, correction) lives in the lanes of that
// query's column.
//
// Reference: PagedAttention::forward, /root/reference/src/models/layers/attention.rs:947-958
// (varlen prefill over cu_seqlens with a cached prefix; decode with split-K, workspace
// /root/reference/src/utils/kvcache_allocator.rs:662-673); golden formula
// /root/reference/tests/probes/compare_flashinfer_probe.py:51-73.
#include "common.h"
#include "qk_row.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ bf16x8 load8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
// A barrier for what went through LDS, written out: this wave's LDS operations are waited for,
// reads of global memory that are under way are not.  `wait_global` is the other half, for a
// wave whose writes to global memory others are about to read.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }
__device__ __forceinline__ void wait_global() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// =====================================================================================
// Decode: every sequence has one query token.  Workgroup (kv head, sequence, split): the
// query heads of the kv group are the columns of one tile; the workgroup's four waves take
// alternate 32-key steps of its chunk of `keys_per_wg` keys and merge through LDS.  A wave keeps loads in flight all the time: the K operands of the next
// step are asked for as soon as the scores of this one are computed, the V operands as soon
// as this step's have been used, into the same registers.  The page numbers of the chunk
// are read once into LDS, so that no step waits for the block table.  Partial results
// (sums scaled by 2^-m, with m and l) go to a workspace, combined by the second kernel in
// split order; with one split for every sequence the kernel writes the result itself.
// =====================================================================================
//
// PACKED: the step's own part of the work is done here too, which saves the kernel that otherwise
// runs before this one.  `q` is then the packed projection [sequences, (nq + 2 nkv) d] (1: bfloat16
// rows; 2: float32 partial sums of a product cut along K): every workgroup norms and rotates its own
// query heads into LDS, and the workgroup whose chunk holds the sequence's last position first does
// the same for the new key, copies the new value, and writes both into the cache, from where it
// reads them back with the rest of its chunk (a workgroup sees its own writes after a barrier; no
// other workgroup of the launch reads that position).  The caches are therefore not `__restrict__`
// nor read-only in this form.
struct PackedStep {
  int slices;                  // PACKED == 2: partial sums, `slice_stride` elements apart
  size_t slice_stride;
  const float* bias;           // of the packed row (float32), or null
  const float* qw;             // per-head norm weights [d], or null (both)
  const float* kw;
  float eps;
  const float* cos_t;          // [positions, rot / 2]
  const float* sin_t;
  int rot, interleaved;
  const int* positions;        // [sequences]
  const long long* slots;      // [sequences]; negative: the sequence's key and value are not stored
};

template <int KC, int DT, int PACKED>
__global__ __launch_bounds__(256, DT > 8 ? 1 : 2) void attn_decode_split_kernel(
    const void* q_v, bf16* k_cache_w, bf16* vt_cache_w,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ ctx_lens,
    float* __restrict__ part_o, float* __restrict__ part_ml, bf16* __restrict__ out, int max_splits, float scale_log2,
    int window, int page, int nq, int nkv, int d, int keys_per_wg, PackedStep ps) {
  extern __shared__ float lds[];  // [4 waves][g][d] + [4][g][2] + page numbers of the chunk
  const bf16* k_cache = k_cache_w;
  const bf16* vt_cache = vt_cache_w;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  // the kv head runs fastest: workgroups go to the chip's eight dies in turn, and with eight kv
  // heads a die then has one head of every sequence and split, the same work as every other die
  // (with the split fastest and an even number of splits, one half of the dies got the full
  // chunks and the other half the sequences' short last ones)
  // Splits are launched in their own order: those past a sequence's end, which end at once, come
  // after everything that has keys.  Launched first (so that the long sequences' last splits would
  // not run alone at the end) they left the workgroups that follow unevenly spread over the compute
  // units wherever about two of those per unit had keys: 16 sequences of 8,500 keys on 8 kv heads in
  // chunks of 2,176 took 134 us in a grid laid out for 16,384 keys against 105 in one for 8,704; in
  // this order 104 either way, and batches of mixed lengths take the same time in both orders.
  const int kvh = blockIdx.x, seq = blockIdx.y, split = blockIdx.z;
  const int g = nq / nkv;
  const int ctx = ctx_lens[seq];
  // asked for together with the length, not after the test below that needs it
  const int tok_pos = PACKED ? ps.positions[seq] : 0;
  const long long slot = PACKED ? ps.slots[seq] : -1;
  const int pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int k_begin = (lo & ~31) + split * keys_per_wg;
  if (k_begin > pos) return;  // no keys for this split (the combine kernel knows)
  const int k_end = min(pos + 1, k_begin + keys_per_wg);  // exclusive

  float* lds_o = lds;                                        // [4][g][d]
  float* lds_ml = lds + 4 * g * d;                           // [4][g][2]
  int* pages = reinterpret_cast<int*>(lds_ml + 4 * g * 2);   // [keys_per_wg / page + 1]
  const int page_shift = __ffs(page) - 1;                    // the page size is a power of two
  const int first_page = k_begin >> page_shift;
  const int n_pages = ((k_end - 1) >> page_shift) - first_page + 1;
  const int* bt = block_tables + (size_t)seq * max_pages;
  for (int i = threadIdx.x; i < n_pages; i += 256) pages[i] = bt[first_page + i];

  // the four waves take alternate steps: the two halves of a 128-byte line of V^T (64 keys) are
  // then asked for at about the same time
  const int kb0 = k_begin + 32 * wave;
  const int kb1 = k_end;

  bf16x8 ka[2][KC], va[DT];
  // K operands of keys k_base..k_base+31: tile 0 row r <-> key k_base + 8*(r/4) + r%4, tile 1
  // that + 4.  Keys past the sequence are read from its last group of 8 (and masked).
  auto load_k = [&](int k_base) {
    int kgrp = k_base + 8 * (r >> 2);
    if (kgrp > pos) kgrp = pos & ~7;
    const int kpage = pages[(kgrp >> page_shift) - first_page];
    const bf16* kp = k_cache + (((size_t)kpage * nkv + kvh) * page + (kgrp & (page - 1)) + (r & 3)) * d;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int off = 32 * c + 8 * j;
      if (off < d) {
        ka[0][c] = load8(kp + off);
        ka[1][c] = load8(kp + 4 * d + off);
      } else {
        ka[0][c] = zero8();
        ka[1][c] = zero8();
      }
    }
  };
  // V^T operands: row 16*dt + r, keys k_base + 8j .. +7 (one group of eight of the pool)
  auto load_v = [&](int k_base) {
    int vgrp = k_base + 8 * j;
    if (vgrp > pos) vgrp = pos & ~7;
    const int vpage = pages[(vgrp >> page_shift) - first_page];
    const bf16* vp = vt_cache + ((size_t)vpage * nkv + kvh) * d * page + ((size_t)((vgrp & (page - 1)) >> 3) * d + r) * 8;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) va[dt] = (16 * dt < d) ? load8(vp + (size_t)16 * dt * 8) : zero8();
  };

  // this lane's query column: head kvh*g + r of the sequence, or none
  const bool col = r < g;
  bf16x8 qb[KC];
  if constexpr (PACKED == 0) {
    const bf16* qrow = reinterpret_cast<const bf16*>(q_v) + ((size_t)seq * nq + kvh * g + (col ? r : 0)) * d;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int off = 32 * c + 8 * j;
      qb[c] = (col && off < d) ? load8(qrow + off) : zero8();
    }
    __syncthreads();
    if (kb0 < kb1) {
      load_k(kb0);
      load_v(kb0);
    }
  } else {
    // The waves share out the heads: in the workgroup that holds the last position the new key
    // and value first, then the group's query heads, which go to LDS (in the space of the merge).
    // The first keys and values are asked for before the heads are worked on, so that what the
    // heads need travels beside them.
    // (Measured at 8 sequences of 4,096 keys, 32 query and 8 kv heads of 128: 30.9 us against 27.8
    // for the kernel that is given q, and the kernel of 4.9 us before it is gone.  Every lane
    // making its own part of the heads in registers, without LDS, took 32.2: each wave then reads
    // the norm's weights and the tables' rows again for all 64 lanes.)
    constexpr bool PARTS = PACKED == 2;
    bf16* qs = reinterpret_cast<bf16*>(lds_o);   // [g][d]
    const int heads = nq + 2 * nkv;
    const bool owner = pos < k_begin + keys_per_wg && slot >= 0;
    const int first_q = owner ? 2 : 0;           // rows: [new key, new value,] query heads
    const int n_rows = g + first_q;
    auto head_of = [&](int row) { return row >= first_q ? kvh * g + row - first_q : row == 0 ? nq + kvh : nq + nkv + kvh; };
    auto packed_head = [&](int h) {
      return PackedHead<bf16, PARTS>{q_v, ((size_t)seq * heads + h) * d, ps.slices, ps.slice_stride,
                                     ps.bias ? ps.bias + (size_t)h * d : nullptr};
    };
    const long long spage = slot >> page_shift;
    const int soff = (int)(slot & (page - 1));
    bf16* k_new = k_cache_w + (((size_t)spage * nkv + kvh) * page + soff) * d;
    bf16* v_new = vt_cache_w + ((size_t)spage * nkv + kvh) * d * page + (size_t)(soff >> 3) * d * 8 + (soff & 7);
    lds_barrier();     // the page numbers are in LDS
    // The first keys and values are asked for before the heads are worked on, except in a chunk so
    // short that a wave's first step holds the new key: that waits until the key is written.
    const bool late = owner && k_end - k_begin <= 128;
    if (!late && kb0 < kb1) {
      load_k(kb0);
      load_v(kb0);
    }
    for (int row = wave; row < n_rows; row += 4) {
      const auto x = packed_head(head_of(row));
      if (row == 1 && owner)
        copy_head<bf16, PARTS>(x, d, lane, v_new, (size_t)8);
      else      // a query head into LDS, or the new key into the cache
        norm_rope_head<bf16, PARTS>(x, row >= first_q ? ps.qw : ps.kw, ps.eps, ps.cos_t, ps.sin_t, ps.rot, ps.interleaved,
                                    tok_pos, d, lane, row >= first_q ? qs + (size_t)(row - first_q) * d : k_new);
    }
    if (owner && wave < 2) wait_global();   // the new key and value are written (what the other waves read comes after the barrier)
    lds_barrier();     // the heads are in LDS
    const bf16* qrow = qs + (size_t)(col ? r : 0) * d;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int off = 32 * c + 8 * j;
      qb[c] = (col && off < d) ? load8(qrow + off) : zero8();
    }
    lds_barrier();     // before the merge's space is written
    if (late && kb0 < kb1) {
      load_k(kb0);
      load_v(kb0);
    }
  }

  f32x4 acc[DT];
#pragma unroll
  for (int dt = 0; dt < DT; ++dt) acc[dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = -INFINITY, l_run = 0.f;   // running max (log2 domain) and this lane's part of the sum
  for (int kb = kb0; kb < kb1; kb += 128) {
    const bool more = kb + 128 < kb1;
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      s0 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[0][c], qb[c], s0, 0, 0, 0);
      s1 = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[1][c], qb[c], s1, 0, 0, 0);
    }
    if (more) load_k(kb + 128);
    float sc[8];
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      sc[v] = s0[v] * scale_log2;
      sc[4 + v] = s1[v] * scale_log2;
    }
    if (kb + 31 > pos || kb < lo) {   // some key of the step is hidden from the query
      const int key0 = kb + 8 * j;
#pragma unroll
      for (int v = 0; v < 8; ++v) {
        const int key = key0 + v;
        if (key > pos || key < lo) sc[v] = -INFINITY;
      }
    }
    float mx = sc[0];
#pragma unroll
    for (int v = 1; v < 8; ++v) mx = fmaxf(mx, sc[v]);
    mx = fmaxf(mx, lane_xor<16>(mx));
    mx = fmaxf(mx, lane_xor<32>(mx));
    const float m_new = fmaxf(m_run, mx);
    const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m_run - m_safe);
    float psum = 0.f;
    bf16x8 pb;
#pragma unroll
    for (int v = 0; v < 8; ++v) {
      const float p = __builtin_amdgcn_exp2f(sc[v] - m_safe);
      psum += p;
      pb[v] = (__bf16)p;
    }
    l_run = l_run * corr + psum;
    m_run = m_new;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      acc[dt][0] *= corr;
      acc[dt][1] *= corr;
      acc[dt][2] *= corr;
      acc[dt][3] *= corr;
      acc[dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va[dt], pb, acc[dt], 0, 0, 0);
    }
    if (more) load_v(kb + 128);
  }
  // the column's sum over the four lane groups
  float lt = l_run + lane_xor<16>(l_run);
  lt += lane_xor<32>(lt);
  if (col) {
    if (j == 0) {
      lds_ml[(wave * g + r) * 2] = m_run;
      lds_ml[(wave * g + r) * 2 + 1] = lt;
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt >= d) break;
      float* o = lds_o + ((size_t)wave * g + r) * d + 16 * dt + 4 * j;
      o[0] = acc[dt][0];
      o[1] = acc[dt][1];
      o[2] = acc[dt][2];
      o[3] = acc[dt][3];
    }
  }
  __syncthreads();
  // merge the four waves, in wave order, and store the partial of (seq, head, split)
  for (int idx = threadIdx.x; idx < g * d; idx += blockDim.x) {
    const int h = idx / d, i = idx - h * d;
    float mm = -INFINITY;
#pragma unroll
    for (int wv = 0; wv < 4; ++wv) mm = fmaxf(mm, lds_ml[(wv * g + h) * 2]);
    float o = 0.f, ll = 0.f;
#pragma unroll
    for (int wv = 0; wv < 4; ++wv) {
      const float mw = lds_ml[(wv * g + h) * 2];
      const float f = (mw == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(mw - mm);
      o += lds_o[((size_t)wv * g + h) * d + i] * f;
      ll += lds_ml[(wv * g + h) * 2 + 1] * f;
    }
    if (max_splits == 1) {   // the only split of every sequence: the result itself
      out[((size_t)seq * nq + kvh * g + h) * d + i] = __float2bfloat16(o * (1.f / ll));   // as the combine rounds
      continue;
    }
    const size_t pidx = ((size_t)seq * nq + kvh * g + h) * max_splits + split;
    part_o[pidx * d + i] = o;
    if (i == 0) {
      part_ml[pidx * 2] = mm;
      part_ml[pidx * 2 + 1] = ll;
    }
  }
}

// One wave per (head, sequence).  Lanes first share out the splits to find the common
// maximum and each split's weight, then every lane sums its output dims over the splits in
// split order.  The kernel lives on latency, so whatever can be asked for at once is: the
// sequence's length, the first 64 splits' (m, l) and the first kEarly splits' sums all start
// before anything is known about them (what lies past the sequence's last split is dropped).
__global__ __launch_bounds__(64) void attn_decode_combine_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ ctx_lens,
    bf16* __restrict__ out, int max_splits, int window, int nq, int d, int keys_per_wg) {
  extern __shared__ float f_s[];  // [max_splits] weight of each split
  constexpr int kEarly = 16;
  const int head = blockIdx.x, seq = blockIdx.y, lane = threadIdx.x;
  const size_t base = ((size_t)seq * nq + head) * max_splits;
  const float* po = part_o + base * d;
  const int ctx = ctx_lens[seq];
  float2 ml0 = {-INFINITY, 0.f};
  if (lane < max_splits) ml0 = *reinterpret_cast<const float2*>(part_ml + (base + lane) * 2);
  float early[2][kEarly];          // output dims lane and lane + 64 of the first splits
#pragma unroll
  for (int c = 0; c < 2; ++c)
#pragma unroll
    for (int e = 0; e < kEarly; ++e)
      early[c][e] = (e < max_splits && lane + 64 * c < d) ? po[(size_t)e * d + lane + 64 * c] : 0.f;
  const int pos = ctx - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int n_splits = (pos - (lo & ~31)) / keys_per_wg + 1;
  float mm = lane < n_splits ? ml0.x : -INFINITY;
  for (int s = lane + kWave; s < n_splits; s += kWave) mm = fmaxf(mm, part_ml[(base + s) * 2]);
  mm = wave_max(mm);
  float ll = 0.f;
  for (int s = lane; s < n_splits; s += kWave) {
    const float ms = s == lane ? ml0.x : part_ml[(base + s) * 2];
    const float ls = s == lane ? ml0.y : part_ml[(base + s) * 2 + 1];
    const float f = __builtin_amdgcn_exp2f(ms - mm);
    f_s[s] = f;
    ll += ls * f;
  }
  ll = wave_sum(ll);
  __syncthreads();
  const float inv = 1.f / ll;
  for (int i = lane, c = 0; i < d; i += kWave, ++c) {
    float o = 0.f;
    int s = 0;
    if (c < 2) {
#pragma unroll
      for (int e = 0; e < kEarly; ++e)
        if (e < n_splits) o += (c == 0 ? early[0][e] : early[1][e]) * f_s[e];
      s = n_splits < kEarly ? n_splits : kEarly;
    }
    for (; s + 4 <= n_splits; s += 4) {
      const float a0 = po[(size_t)s * d + i], a1 = po[(size_t)(s + 1) * d + i], a2 = po[(size_t)(s + 2) * d + i],
                  a3 = po[(size_t)(s + 3) * d + i];
      o += a0 * f_s[s];
      o += a1 * f_s[s + 1];
      o += a2 * f_s[s + 2];
      o += a3 * f_s[s + 3];
    }
    for (; s < n_splits; ++s) o += po[(size_t)s * d + i] * f_s[s];
    out[((size_t)seq * nq + head) * d + i] = __float2bfloat16(o * inv);
  }
}

// The same for many splits (a long context of few sequences: 513 splits at 131,072 keys), where
// one wave's walk over the splits takes longer than the attention itself: sixteen waves per
// (head, sequence).  All threads share out the splits for the common maximum and the weights;
// wave w then sums splits [w c, (w + 1) c), c = ceil(splits / 16), in split order, four splits
// of loads in flight, and the sixteen sums are added in wave order.  The order depends on the
// number of splits alone.
constexpr int kWideWaves = 16;
constexpr int kCombineWideFrom = 24;           // launches with more splits than this take the wide kernel
__global__ __launch_bounds__(64 * kWideWaves) void attn_decode_combine_wide_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ ctx_lens,
    bf16* __restrict__ out, int max_splits, int window, int nq, int d, int keys_per_wg) {
  extern __shared__ float f_s[];                 // [max_splits] weights | [16][d] sums of the waves | [16] | [16]
  float* o_w = f_s + max_splits;
  float* red_m = o_w + kWideWaves * d;
  float* red_l = red_m + kWideWaves;
  const int head = blockIdx.x, seq = blockIdx.y, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t base = ((size_t)seq * nq + head) * max_splits;
  const float* po = part_o + base * d;
  const int pos = ctx_lens[seq] - 1;
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int n_splits = (pos - (lo & ~31)) / keys_per_wg + 1;
  float mm = -INFINITY;
  for (int s = tid; s < n_splits; s += 64 * kWideWaves) mm = fmaxf(mm, part_ml[(base + s) * 2]);
  mm = wave_max(mm);
  if (lane == 0) red_m[wave] = mm;
  __syncthreads();
  mm = red_m[0];
#pragma unroll
  for (int w = 1; w < kWideWaves; ++w) mm = fmaxf(mm, red_m[w]);
  float ll = 0.f;
  for (int s = tid; s < n_splits; s += 64 * kWideWaves) {
    const float2 ml = *reinterpret_cast<const float2*>(part_ml + (base + s) * 2);
    const float f = __builtin_amdgcn_exp2f(ml.x - mm);
    f_s[s] = f;
    ll += ml.y * f;
  }
  ll = wave_sum(ll);
  if (lane == 0) red_l[wave] = ll;
  __syncthreads();
  ll = 0.f;
#pragma unroll
  for (int w = 0; w < kWideWaves; ++w) ll += red_l[w];
  const int chunk = (n_splits + kWideWaves - 1) / kWideWaves;
  const int s0 = wave * chunk, s1 = min(s0 + chunk, n_splits);
  float o[4] = {0.f, 0.f, 0.f, 0.f};             // output dims lane + 64 c (head sizes up to 256)
  for (int s = s0; s < s1; s += 4) {
    float a[4][4];
#pragma unroll
    for (int u = 0; u < 4; ++u)
#pragma unroll
      for (int c = 0; c < 4; ++c)
        a[u][c] = (s + u < s1 && lane + 64 * c < d) ? po[(size_t)(s + u) * d + lane + 64 * c] : 0.f;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float f = s + u < s1 ? f_s[s + u] : 0.f;
#pragma unroll
      for (int c = 0; c < 4; ++c) o[c] += a[u][c] * f;
    }
  }
#pragma unroll
  for (int c = 0; c < 4; ++c)
    if (lane + 64 * c < d) o_w[wave * d + lane + 64 * c] = o[c];
  __syncthreads();
  const float inv = 1.f / ll;
  for (int i = tid; i < d; i += 64 * kWideWaves) {
    float t = 0.f;
#pragma unroll
    for (int w = 0; w < kWideWaves; ++w) t += o_w[w * d + i];
    out[((size_t)seq * nq + head) * d + i] = __float2bfloat16(t * inv);
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// Sizes the MFMA kernels take: head_dim a multiple of 16 up to 256, page size a power of two
// of at least 8, at most 16 query heads per kv head (decode).  Returns 1 if supported.
int xi_attention_mfma_supported(int nq, int nkv, int d, int page) {
  return (d % 16 == 0 && d >= 16 && d <= 256 && page >= 8 && (page & (page - 1)) == 0 && nq % nkv == 0) ? 1 : 0;
}

// The decode launch: `packed` 0 takes q [sequences, nq, d]; 1 and 2 the packed projection, see PackedStep.
static int launch_decode(int packed, const void* q, const PackedStep& ps, void* k_cache, void* vt_cache,
                         const int* block_tables, int max_pages, const int* ctx_lens, void* out, float* part_o,
                         float* part_ml, int max_splits, int keys_per_wg, float scale, int window, int page, int n_seq,
                         int nq, int nkv, int d, hipStream_t stream) {
  XI_CHECK(xi_attention_mfma_supported(nq, nkv, d, page), "attention_decode: unsupported sizes nq=%d nkv=%d d=%d page=%d",
           nq, nkv, d, page);
  const int g = nq / nkv;
  XI_CHECK(g <= 16, "attention_decode: %d query heads per kv head exceed 16", g);
  XI_CHECK(keys_per_wg > 0 && keys_per_wg % 128 == 0, "attention_decode: keys_per_wg %d must be a multiple of 128", keys_per_wg);
  XI_CHECK(max_splits > 0 && nkv <= 65535 && n_seq <= 65535, "attention_decode: bad grid");
  XI_CHECK((size_t)max_splits * sizeof(float) <= 48 * 1024, "attention_decode: %d splits are too many", max_splits);
  const size_t lds = (size_t)(4 * g * d + 4 * g * 2) * sizeof(float) + (size_t)(keys_per_wg / page + 2) * sizeof(int);
  XI_CHECK(lds <= 64 * 1024, "attention_decode: group %d x head_dim %d needs too much LDS", g, d);
  if (n_seq == 0) return 0;
  dim3 grid(nkv, n_seq, max_splits);
  const float sl = scale * kLog2e;
#define XI_DC(KC, DT, PACKED)                                                                      \
  attn_decode_split_kernel<KC, DT, PACKED><<<grid, 256, lds, stream>>>(                            \
      q, (bf16*)k_cache, (bf16*)vt_cache, block_tables, max_pages, ctx_lens,                       \
      part_o, part_ml, (bf16*)out, max_splits, sl, window, page, nq, nkv, d, keys_per_wg, ps)
#define XI_DCP(KC, DT)             \
  do {                             \
    if (packed == 0) XI_DC(KC, DT, 0); \
    else if (packed == 1) XI_DC(KC, DT, 1); \
    else XI_DC(KC, DT, 2);         \
  } while (0)
  if (d <= 64) XI_DCP(2, 4);
  else if (d <= 128) XI_DCP(4, 8);
  else XI_DCP(8, 16);
#undef XI_DCP
#undef XI_DC
  XI_LAUNCH_CHECK("attention_decode_split");
  if (max_splits == 1) return 0;   // the split kernel has written the result
  if (max_splits > kCombineWideFrom) {
    const size_t wide_lds = (size_t)(max_splits + kWideWaves * d + 2 * kWideWaves) * sizeof(float);
    XI_CHECK(wide_lds <= 64 * 1024, "attention_decode: %d splits of head_dim %d are too many", max_splits, d);
    attn_decode_combine_wide_kernel<<<dim3(nq, n_seq), 64 * kWideWaves, wide_lds, stream>>>(
        part_o, part_ml, ctx_lens, (bf16*)out, max_splits, window, nq, d, keys_per_wg);
  } else {
    attn_decode_combine_kernel<<<dim3(nq, n_seq), 64, max_splits * sizeof(float), stream>>>(
        part_o, part_ml, ctx_lens, (bf16*)out, max_splits, window, nq, d, keys_per_wg);
  }
  XI_LAUNCH_CHECK("attention_decode_combine");
  return 0;
}

int xi_attention_decode_bf16(const void* q, const void* k_cache, const void* vt_cache, const int* block_tables,
                             int max_pages, const int* ctx_lens, void* out, float* part_o, float* part_ml,
                             int max_splits, int keys_per_wg, float scale, int window, int page, int n_seq,
                             int nq, int nkv, int d, hipStream_t stream) {
  return launch_decode(0, q, PackedStep{}, const_cast<void*>(k_cache), const_cast<void*>(vt_cache), block_tables,
                       max_pages, ctx_lens, out, part_o, part_ml, max_splits, keys_per_wg, scale, window, page, n_seq,
                       nq, nkv, d, stream);
}

// A decode step's attention from the packed projection: per-head norm and rotation of q and k,
// the new keys and values into the cache at `slots`, and the attention over the cache, in one
// launch (plus the combine).  `qkv` is [n_seq, (nq + 2 nkv) d] bfloat16 (`slices` 0) or `slices`
// float32 partial sums of that shape, added in slice order.  The other operands are those of
// xi_qk_norm_rope_kv and xi_attention_decode_bf16, and the results have the same bits as theirs.
int xi_attention_decode_packed_bf16(const void* qkv, int slices, const float* bias, const float* qw, const float* kw,
                                    float eps, const float* cos_t, const float* sin_t, int rot, int interleaved,
                                    const int* positions, const long long* slots, void* k_cache, void* vt_cache,
                                    const int* block_tables, int max_pages, const int* ctx_lens, void* out,
                                    float* part_o, float* part_ml, int max_splits, int keys_per_wg, float scale,
                                    int window, int page, int n_seq, int nq, int nkv, int d, hipStream_t stream) {
  XI_CHECK(rot >= 0 && rot <= d && rot % 2 == 0, "attention_decode_packed: rotary_dim %d must be even and <= head_dim %d", rot, d);
  XI_CHECK((qw == nullptr) == (kw == nullptr), "attention_decode_packed: q and k norm weights must both be given or both absent");
  XI_CHECK(slices >= 0 && slices <= 64, "attention_decode_packed: %d slices", slices);
  PackedStep ps;
  ps.slices = slices;
  ps.slice_stride = (size_t)n_seq * (nq + 2 * nkv) * d;
  ps.bias = bias;
  ps.qw = qw;
  ps.kw = kw;
  ps.eps = eps;
  ps.cos_t = cos_t;
  ps.sin_t = sin_t;
  ps.rot = rot;
  ps.interleaved = interleaved;
  ps.positions = positions;
  ps.slots = slots;
  return launch_decode(slices ? 2 : 1, qkv, ps, k_cache, vt_cache, block_tables, max_pages, ctx_lens, out, part_o,
                       part_ml, max_splits, keys_per_wg, scale, window, page, n_seq, nq, nkv, d, stream);
}

}  // extern "C"
