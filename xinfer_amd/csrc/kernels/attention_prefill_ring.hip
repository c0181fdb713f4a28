// bfloat16 paged causal GQA attention for prompt portions on the gfx950 matrix cores, with the
// K and V^T tiles brought into a ring of LDS stages by loads that write LDS themselves.
//
// The arithmetic, the layout of scores (S^T = K . Q^T, a query's scores in the lanes of its
// column), the column tiles of a wave and the softmax are those of attention_prefill.hip; what
// differs is how a tile of 64 keys reaches LDS.  There a thread loads 16-byte chunks into registers
// and stores them to LDS one tile ahead; a workgroup that runs alone on its compute unit (the
// longest query block of a short prompt) then waits a memory round trip per tile.  Here every lane
// of a wave asks for one 16-byte chunk with `global_load_lds_dwordx4`, whose 64 results land in
// 1 KB of consecutive LDS; no register holds them, so S - 1 tiles can be in flight for a ring of S
// stages, and a tile is waited for with a count (`s_waitcnt vmcnt`), not by draining the queue.
//
// Since a load's 64 chunks land side by side, rows cannot be padded against bank conflicts; the
// chunks of a row are permuted instead.  K rows (32 * KC elements): chunk ch of row p sits at
// position ch ^ x(p), x(p) = (p >> sh) & (min(4 * KC, 16) - 1) with sh so that 16 consecutive rows
// differ in x or in their 256-byte phase.  V^T rows (64 keys): chunk cc of row dd at position
// cc ^ ((dd >> 1) & 7).  Each lane picks the global chunk that belongs at its place.  As in
// attention_prefill.hip the keys of a 32-key step are permuted over the rows:
// key k sits at row 16*((k>>2)&1) + 4*(k>>3) + (k&3).
//
// Head sizes 32, 64, 128 and 256 (whole 32-wide steps of the matrix product and a power of two
// of chunks a row); other sizes stay with attention_prefill.hip.
//
// Reference: PagedAttention::forward prefill branch,
// /root/reference/src/models/layers/attention.rs:947-958; golden formula
// /root/reference/tests/probes/compare_flashinfer_probe.py:51-73.
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace ring {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int kKeys = 64;      // keys per tile (two steps of 32)
constexpr float kSlack = 8.f;  // how far (log2) a score may exceed the softmax reference point

__device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zero8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// One 16-byte chunk per lane from global memory to LDS at `lds_addr` (the same in all lanes) +
// 16 * lane.  The compiler does not see that LDS is written: whoever reads it waits for the load
// with an explicit vmcnt and a barrier first.
__device__ __forceinline__ void load_lds16(const void* g, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(g), "s"(lds_addr) : "memory", "m0");
}

// The same with the address as a base that is the same in all lanes plus a byte offset per lane.
__device__ __forceinline__ void load_lds16(const void* base, unsigned lane_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
}

// vmcnt(n), the other counters untouched (gfx9 encoding: vmcnt in bits 3:0 and 15:14)
template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

// KS = 2: two groups of waves own the same column tiles and take one 32-key step of a tile each;
// the second group's sums are merged into the first's through LDS at the end.
// BIGPAGE: a page holds at least a tile's 64 keys (and tiles start at multiples of 64), so a tile
// lies in one page: its page number is one scalar lookup and every lane's address the tile's base
// plus an offset that never changes; with smaller pages every chunk looks its page up.
template <int KC, int NQT, int GH, int NWV, int KS, int S, bool BIGPAGE>
__global__ __launch_bounds__(64 * NWV, 2) void attn_prefill_ring_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ vt_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tiles,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, bf16* __restrict__ out, float scale_log2,
    int window, int page_shift, int nq, int nkv) {
  constexpr int D = 32 * KC, DT = 2 * KC;
  constexpr int NT = 64 * NWV, WPG = NWV / KS;
  constexpr int QB = 16 * (WPG * NQT / GH);       // query positions per workgroup
  static_assert(NWV % KS == 0 && (KS == 1 || KS == 2), "one or two groups of waves");
  static_assert((WPG * NQT) % GH == 0, "tiles must divide into whole position blocks");
  static_assert(KC == 1 || KC == 2 || KC == 4 || KC == 8, "a power of two of chunks a row");
  constexpr int KBYTES = kKeys * D * 2, VBYTES = D * kKeys * 2, STAGE = KBYTES + VBYTES;
  constexpr int KI = KBYTES / 1024, VI = VBYTES / 1024;     // wave-wide loads of a tile: K, then V^T
  static_assert((KI + VI) % NWV == 0, "every wave issues the same number of loads a tile");
  constexpr int LPW = (KI + VI) / NWV;                      // loads a wave issues for a tile
  static_assert((S - 1) * LPW < 64 && S >= 2, "the tiles in flight must fit the load counter");
  constexpr int CPK = 4 * KC;                               // chunks of a K row
  constexpr int XM = (CPK < 16 ? CPK : 16) - 1;             // mask of the permutation of a K row's chunks
  constexpr int XS = CPK >= 16 ? 0 : (CPK == 8 ? 1 : 2);    // rows that share a 256-byte phase differ in x
  extern __shared__ __align__(1024) unsigned char smem[];
  int* bt_s = reinterpret_cast<int*>(smem + (size_t)S * STAGE);      // [max_pages]
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave_abs = tid >> 6;
  const int wave = wave_abs % WPG, grp = wave_abs / WPG;     // the wave within its group, and the group
  const int r = lane & 15, j = lane >> 4;
  const int page = 1 << page_shift;
  const int g = nq / nkv, groups = g / GH;
  const int kvh = blockIdx.x / groups;
  const int h0 = kvh * g + (blockIdx.x - kvh * groups) * GH;
  const size_t kv_head_stride = (size_t)D << page_shift;     // elements of one (page, kv head) block

  // ---- what this lane brings of every tile: per load of its wave the key (K) or the row and the
  // first key (V^T) of its chunk, and where the chunk starts within the row
  int ld_key[LPW], ld_off[LPW];       // K: key within the tile, element offset 8 * ch; V^T: first key of the chunk, row
  unsigned ld_dst[LPW];               // byte offset of the load's 1 KB within a stage
#pragma unroll
  for (int t = 0; t < LPW; ++t) {
    const int ii = wave_abs + NWV * t;
    ld_dst[t] = ii * 1024;
    if (ii < KI) {
      const int off = ii * 1024 + lane * 16;
      const int p = off / (2 * D), pos = (off % (2 * D)) / 16;
      const int ch = pos ^ ((p >> XS) & XM);
      const int p32 = p & 31, rest = p32 & 15;
      ld_key[t] = (p & 32) + 8 * (rest >> 2) + 4 * (p32 >> 4) + (rest & 3);
      ld_off[t] = 8 * ch;
    } else {
      const int off = (ii - KI) * 1024 + lane * 16;
      const int dd = off / 128, pos = (off % 128) / 16;
      ld_key[t] = 8 * (pos ^ ((dd >> 1) & 7));
      ld_off[t] = dd;
    }
  }

  unsigned ld_lane[LPW];              // BIGPAGE: byte offset of the lane's chunk from the tile's first key in its page
#pragma unroll
  for (int t = 0; t < LPW; ++t) {
    const int ii = wave_abs + NWV * t;
    ld_lane[t] = ii < KI ? 2u * (unsigned)(ld_key[t] * D + ld_off[t])
                         : 2u * (unsigned)(((ld_key[t] >> 3) * D + ld_off[t]) * 8);      // V: [offset / 8, d, 8]
  }
  // where this lane reads the matrix operands within a stage (bytes): K rows r and 16 + r of a step,
  // chunk 4c + j at its permuted place; V^T rows 16 dt + r, chunk 4 sub + j at its permuted place.
  // What depends on c or sub through the permutation is kept per c or sub; steps, halves and dt
  // are constant offsets.
  unsigned k_rd[KC], v_rd[2];
#pragma unroll
  for (int c = 0; c < KC; ++c) k_rd[c] = 2u * (unsigned)(r * D + 8 * ((4 * c + j) ^ ((r >> XS) & XM)));
#pragma unroll
  for (int sub = 0; sub < 2; ++sub) v_rd[sub] = 2u * (unsigned)(r * kKeys + 8 * ((4 * sub + j) ^ ((r >> 1) & 7)));
  static_assert(((16 >> XS) & XM) == 0 && ((32 >> XS) & XM) == 0, "rows 16 and 32 further on keep their permutation");

  const int seq = tiles[2 * blockIdx.y], q0_blk = tiles[2 * blockIdx.y + 1];
  const int q_begin = cu_q[seq], q_len = cu_q[seq + 1] - q_begin;
  const int ctx = ctx_lens[seq];
  const int pos0 = ctx - q_len;         // position of the portion's first token
  const int k_last = ctx - 1;
  {
    const int* bt = block_tables + (size_t)seq * max_pages;
    const int n_pages = (k_last + page) / page;    // pages that hold keys 0..k_last
    for (int i = threadIdx.x; i < n_pages; i += NT) bt_s[i] = bt[i];
  }

  // keys the workgroup walks
  const int wg_nq = min(QB, q_len - q0_blk);
  const int wg_first = pos0 + q0_blk, wg_last = wg_first + wg_nq - 1;
  const int wg_lo = (window > 0 && wg_first - window + 1 > 0) ? wg_first - window + 1 : 0;
  const int k_begin = wg_lo & ~(kKeys - 1);

  // this wave's queries: the position blocks its tiles lie in
  const int pb_lo = (wave * NQT) / GH, pb_hi = (wave * NQT + NQT - 1) / GH;
  const int q0 = q0_blk + 16 * pb_lo;
  const bool active = q0 < q_len;
  const int n_q = active ? min(16 * (pb_hi - pb_lo + 1), q_len - q0) : 0;
  const int first_pos = pos0 + q0, last_pos = first_pos + n_q - 1;
  const int lo_first = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  const int lo_last = (window > 0 && last_pos - window + 1 > 0) ? last_pos - window + 1 : 0;
  const int wave_k_begin = lo_first & ~31;

  bf16x8 qb[NQT][KC];
  f32x4 acc[DT][NQT];
  float m_run[NQT], l_run[NQT];
  int qpos[NQT], qlo[NQT];
#pragma unroll
  for (int ct = 0; ct < NQT; ++ct) {
    const int tile = wave * NQT + ct;
    const int pb = tile / GH, hh = tile - pb * GH;
    const int qi = q0_blk + 16 * pb + r;
    const bool ok = active && qi < q_len;
    qpos[ct] = ok ? pos0 + qi : -1;
    qlo[ct] = (ok && window > 0 && qpos[ct] - window + 1 > 0) ? qpos[ct] - window + 1 : 0;
    const bf16* qrow = q + ((size_t)(q_begin + (ok ? qi : 0)) * nq + h0 + hh) * D;
#pragma unroll
    for (int c = 0; c < KC; ++c) qb[ct][c] = ok ? ld8(qrow + 32 * c + 8 * j) : zero8();
    m_run[ct] = -INFINITY;
    l_run[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // Asks for the tile of keys kb .. kb + 63 into stage `st`.  Keys past the last one are read
  // from the last one's place (they are masked); tiles past the workgroup's last are asked for
  // all the same, so that the number of loads in flight does not depend on where the walk is.
  const int last_tile = k_last & ~(kKeys - 1);
  auto fetch = [&](int kb, int st) {
    const unsigned base = lds0 + (unsigned)st * STAGE;
    if (BIGPAGE) {
      kb = kb > last_tile ? last_tile : kb;        // a tile past the end: the last one again (nobody reads it)
      const int pid = __builtin_amdgcn_readfirstlane(bt_s[kb >> page_shift]);
      const size_t blk = ((size_t)pid * nkv + kvh) * kv_head_stride;
      const bf16* kbase = k_cache + blk + (size_t)(kb & (page - 1)) * D;
      const bf16* vbase = vt_cache + blk + (size_t)((kb & (page - 1)) >> 3) * D * 8;
#pragma unroll
      for (int t = 0; t < LPW; ++t) {
        const int ii = wave_abs + NWV * t;
        // (which of the two a wave's t-th load takes is the same in all its lanes: made a scalar by hand)
        const unsigned long long a = (unsigned long long)(uintptr_t)(ii < KI ? kbase : vbase);
        const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
        load_lds16(reinterpret_cast<const void*>((uintptr_t)(((unsigned long long)hi << 32) | lo)), ld_lane[t],
                   __builtin_amdgcn_readfirstlane(base + ld_dst[t]));
      }
      return;
    }
#pragma unroll
    for (int t = 0; t < LPW; ++t) {
      const int ii = wave_abs + NWV * t;
      const bf16* src;
      if (ii < KI) {
        int key = kb + ld_key[t];
        key = key > k_last ? k_last : key;
        const int kp = bt_s[key >> page_shift];
        src = k_cache + ((size_t)kp * nkv + kvh) * kv_head_stride + (size_t)(key & (page - 1)) * D + ld_off[t];
      } else {
        int key0 = kb + ld_key[t];
        key0 = key0 > k_last ? (k_last & ~7) : key0;
        const int vp = bt_s[key0 >> page_shift];
        src = vt_cache + ((size_t)vp * nkv + kvh) * kv_head_stride + ((size_t)((key0 & (page - 1)) >> 3) * D + ld_off[t]) * 8;
      }
      load_lds16(src, __builtin_amdgcn_readfirstlane(base + ld_dst[t]));
    }
  };

  __syncthreads();   // the block table is in LDS
  // the queries have landed before the first tile is asked for: from here on the tiles' loads are
  // the only ones in flight, and the counts they are waited for with mean what they say
  wait_loads<0>();
#pragma unroll
  for (int p = 0; p < S - 1; ++p) fetch(k_begin + kKeys * p, p);
  int st = 0;
  for (int kt = k_begin; kt <= wg_last; kt += kKeys) {
    wait_loads<(S - 2) * LPW>();     // this wave's loads of the tile have landed (and its queries)
    __syncthreads();                 // everybody's have; and nobody reads the tile before any more
    fetch(kt + kKeys * (S - 1), st == 0 ? S - 1 : st - 1);
    const unsigned char* Kt = smem + (size_t)st * STAGE;
    const unsigned char* Vt = Kt + KBYTES;
#pragma unroll
    for (int sub = 0; sub < kKeys / 32; ++sub) {
    const int kb = kt + 32 * sub;
    if ((KS == 1 || sub == grp) && active && kb >= wave_k_begin && kb <= last_pos) {
      // a step needs the mask unless every key is at or before every query and inside every window
      const bool masked = (kb + 31 > first_pos) || (kb < lo_last);
      bf16x8 ka[2][KC];
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        ka[0][c] = ld8(reinterpret_cast<const bf16*>(Kt + k_rd[c] + 2 * D * (32 * sub)));
        ka[1][c] = ld8(reinterpret_cast<const bf16*>(Kt + k_rd[c] + 2 * D * (32 * sub + 16)));
      }
      // ---- all scores of the step first
      f32x4 s0[NQT], s1[NQT];
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        s0[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
        s1[ct] = f32x4{0.f, 0.f, 0.f, 0.f};
      }
#pragma unroll
      for (int c = 0; c < KC; ++c)
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct) {
          s0[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[0][c], qb[ct][c], s0[ct], 0, 0, 0);
          s1[ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka[1][c], qb[ct][c], s1[ct], 0, 0, 0);
        }
      if (masked) {
        const int key0 = kb + 8 * j;
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct)
#pragma unroll
          for (int v = 0; v < 4; ++v) {
            if (key0 + v > qpos[ct] || key0 + v < qlo[ct]) s0[ct][v] = -INFINITY;
            if (key0 + 4 + v > qpos[ct] || key0 + 4 + v < qlo[ct]) s1[ct][v] = -INFINITY;
          }
      }
      // ---- the reference point of the exponentials moves only when a score exceeds it by more
      // than 2^kSlack (see attention_prefill.hip); one test for all column tiles
      float mx[NQT];
      bool moved = false;
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        mx[ct] = fmaxf(fmaxf(fmaxf(s0[ct][0], s0[ct][1]), fmaxf(s0[ct][2], s0[ct][3])),
                       fmaxf(fmaxf(s1[ct][0], s1[ct][1]), fmaxf(s1[ct][2], s1[ct][3]))) * scale_log2;
        moved = moved || (mx[ct] > m_run[ct] + kSlack);
      }
      if (__any(moved)) {
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct) {
          float mc = mx[ct];
          mc = fmaxf(mc, lane_xor<16>(mc));
          mc = fmaxf(mc, lane_xor<32>(mc));
          const float m_new = fmaxf(m_run[ct], mc);
          const float corr = (m_new == -INFINITY) ? 1.f : __builtin_amdgcn_exp2f(m_run[ct] - m_new);
          l_run[ct] *= corr;
#pragma unroll
          for (int dt = 0; dt < DT; ++dt) {
            acc[dt][ct][0] *= corr;
            acc[dt][ct][1] *= corr;
            acc[dt][ct][2] *= corr;
            acc[dt][ct][3] *= corr;
          }
          m_run[ct] = m_new;
        }
      }
      // ---- exponentials, then the products with V^T: straight-line code
      bf16x8 pb_[NQT];
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        const float m_safe = (m_run[ct] == -INFINITY) ? 0.f : m_run[ct];
        float psum = 0.f;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float p0 = __builtin_amdgcn_exp2f(fmaf(s0[ct][v], scale_log2, -m_safe));
          const float p1 = __builtin_amdgcn_exp2f(fmaf(s1[ct][v], scale_log2, -m_safe));
          psum += p0 + p1;
          pb_[ct][v] = (__bf16)p0;
          pb_[ct][4 + v] = (__bf16)p1;
        }
        l_run[ct] += psum;
      }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        const bf16x8 va = ld8(reinterpret_cast<const bf16*>(Vt + v_rd[sub] + 2 * kKeys * (16 * dt)));
#pragma unroll
        for (int ct = 0; ct < NQT; ++ct)
          acc[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb_[ct], acc[dt][ct], 0, 0, 0);
      }
    }
    }
    st = st + 1 == S ? 0 : st + 1;
  }
  // the tiles asked for past the end are still on their way into LDS: nothing may be written
  // there (the merge below) before they landed
  wait_loads<0>();
  __syncthreads();

  if (KS == 2) {
    // the second group hands its reference points, sums and accumulators to the first through LDS;
    // both have their column tiles in the same lanes.  Per wave and lane: NQT * (2 + 4 * DT) floats.
    float* xs = reinterpret_cast<float*>(smem) + (size_t)(wave * 64 + lane) * (NQT * (2 + 4 * DT));
    if (grp == 1 && active) {
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        float* x = xs + ct * (2 + 4 * DT);
        x[0] = m_run[ct];
        x[1] = l_run[ct];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          x[2 + 4 * dt] = acc[dt][ct][0];
          x[3 + 4 * dt] = acc[dt][ct][1];
          x[4 + 4 * dt] = acc[dt][ct][2];
          x[5 + 4 * dt] = acc[dt][ct][3];
        }
      }
    }
    __syncthreads();
    if (grp == 0 && active) {
#pragma unroll
      for (int ct = 0; ct < NQT; ++ct) {
        const float* x = xs + ct * (2 + 4 * DT);
        const float m1 = x[0], l1 = x[1];
        const float m = fmaxf(m_run[ct], m1);
        const float c0 = (m_run[ct] == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m_run[ct] - m);
        const float c1 = (m1 == -INFINITY) ? 0.f : __builtin_amdgcn_exp2f(m1 - m);
        l_run[ct] = l_run[ct] * c0 + l1 * c1;
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          acc[dt][ct][0] = acc[dt][ct][0] * c0 + x[2 + 4 * dt] * c1;
          acc[dt][ct][1] = acc[dt][ct][1] * c0 + x[3 + 4 * dt] * c1;
          acc[dt][ct][2] = acc[dt][ct][2] * c0 + x[4 + 4 * dt] * c1;
          acc[dt][ct][3] = acc[dt][ct][3] * c0 + x[5 + 4 * dt] * c1;
        }
      }
    }
  }
  if (active && grp == 0) {
#pragma unroll
    for (int ct = 0; ct < NQT; ++ct) {
      float lt = l_run[ct] + lane_xor<16>(l_run[ct]);
      lt += lane_xor<32>(lt);
      const int tile = wave * NQT + ct;
      const int pb = tile / GH, hh = tile - pb * GH;
      const int qi = q0_blk + 16 * pb + r;
      if (qi >= q_len) continue;
      const float inv = 1.f / lt;
      bf16* o = out + ((size_t)(q_begin + qi) * nq + h0 + hh) * D;
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        bf16* op = o + 16 * dt + 4 * j;
        const f32x4 a = acc[dt][ct];
        op[0] = __float2bfloat16(a[0] * inv);
        op[1] = __float2bfloat16(a[1] * inv);
        op[2] = __float2bfloat16(a[2] * inv);
        op[3] = __float2bfloat16(a[3] * inv);
      }
    }
  }
}

}  // namespace ring
}  // namespace xi

using namespace xi;

extern "C" {

int xi_attention_mfma_supported(int nq, int nkv, int d, int page);
int xi_attention_prefill_block(int d, int g, int small);

// Whether the ring kernel takes a head size (the other conditions are those of the matrix-core kernels).
int xi_attention_prefill_ring_supported(int d) { return d == 32 || d == 64 || d == 128 || d == 256; }

// The same interface as xi_attention_prefill_bf16 (attention_prefill.hip) and the same shapes:
// small = 0: eight waves, the query block of xi_attention_prefill_block(d, g, 0); 1: four waves, half the
// block; 2: eight waves in two groups that split a tile's keys, the block of shape 1.
int xi_attention_prefill_ring_bf16(const void* q, const void* k_cache, const void* vt_cache, const int* block_tables,
                                   int max_pages, const int* tiles, int n_tiles, const int* cu_q, const int* ctx_lens,
                                   void* out, float scale, int window, int page, int nq, int nkv, int d, int small,
                                   hipStream_t stream) {
  XI_CHECK(xi_attention_mfma_supported(nq, nkv, d, page) && xi_attention_prefill_ring_supported(d),
           "attention_prefill_ring: unsupported sizes nq=%d nkv=%d d=%d page=%d", nq, nkv, d, page);
  XI_CHECK(n_tiles >= 0 && n_tiles <= 65535, "attention_prefill_ring: %d query blocks are too many for one launch",
           n_tiles);
  XI_CHECK(small >= 0 && small <= 2, "attention_prefill_ring: unknown workgroup shape %d", small);
  if (n_tiles == 0) return 0;
  const int g = nq / nkv;
  const int gh = g % 4 == 0 ? 4 : (g % 2 == 0 ? 2 : 1);
  dim3 grid(nkv * (g / gh), n_tiles);
  const float sl = scale * ring::kLog2e;
  XI_CHECK(sl > 0.f, "attention_prefill_ring: the scale must be positive");
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if ((1 << b) == page) page_shift = b;
  XI_CHECK(page_shift >= 3, "attention_prefill_ring: the page size %d must be a power of two of at least 8", page);
#define XI_RING(KC, NQT, GH, NWV, KS, S)                                                                      \
  do {                                                                                                        \
    auto kern = page >= ring::kKeys ? ring::attn_prefill_ring_kernel<KC, NQT, GH, NWV, KS, S, true>           \
                                    : ring::attn_prefill_ring_kernel<KC, NQT, GH, NWV, KS, S, false>;         \
    const size_t stages = (size_t)(S) * 2 * ring::kKeys * 32 * KC * 2;                                        \
    const size_t lds = stages + (size_t)max_pages * sizeof(int);                                              \
    XI_CHECK(lds <= 160 * 1024, "attention_prefill_ring: block tables of %d pages do not fit in LDS", max_pages); \
    XI_CHECK(KS == 1 || (size_t)(NWV / KS) * 64 * NQT * (2 + 8 * KC) * sizeof(float) <= stages,               \
             "attention_prefill_ring: the groups' merge does not fit the stages (d=%d)", d);                  \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds); \
    XI_CHECK(e == hipSuccess, "attention_prefill_ring: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e)); \
    kern<<<grid, 64 * NWV, lds, stream>>>((const bf16*)q, (const bf16*)k_cache, (const bf16*)vt_cache, block_tables, \
                                          max_pages, tiles, cu_q, ctx_lens, (bf16*)out, sl, window, page_shift, nq, \
                                          nkv);                                                               \
  } while (0)
#define XI_RING_GH(KC, NQT, NWV, KS, S)                  \
  do {                                                   \
    if (gh == 4) XI_RING(KC, NQT, 4, NWV, KS, S);        \
    else if (gh == 2) XI_RING(KC, NQT, 2, NWV, KS, S);   \
    else XI_RING(KC, NQT, 1, NWV, KS, S);                \
  } while (0)
  // stages: as many as leave the compute unit's 160 KB to the workgroups that share it (two of the
  // four-wave shape, one of the others) beside the block table
#define XI_RING_D(KC, NQT, S8, S4)                       \
  do {                                                   \
    if (small == 2) XI_RING_GH(KC, NQT, 8, 2, S8);       \
    else if (small == 1) XI_RING_GH(KC, NQT, 4, 1, S4);  \
    else XI_RING_GH(KC, NQT, 8, 1, S8);                  \
  } while (0)
  if (d == 32) XI_RING_D(1, 2, 4, 4);
  else if (d == 64) XI_RING_D(2, 2, 4, 4);
  else if (d == 128) XI_RING_D(4, 2, 4, 2);
  else XI_RING_D(8, 1, 2, 2);
#undef XI_RING_D
#undef XI_RING_GH
#undef XI_RING
  XI_LAUNCH_CHECK("attention_prefill_ring");
  return 0;
}

}  // extern "C"
