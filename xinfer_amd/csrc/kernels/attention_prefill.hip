// bfloat16 paged causal GQA attention for prompt portions (and any mixed batch) on the
// gfx950 matrix cores, with K and V^T tiles staged through LDS.
//
// A workgroup of four waves owns a block of consecutive query positions of one sequence
// and GH query heads that share one kv head.  It walks the keys those queries can see in
// tiles of 64: all 256 threads copy the K tile [64 keys, d] and the V^T tile [d, 64 keys]
// from the paged cache into LDS (double buffered; the next tile's global loads are in
// flight while the current one is multiplied, and the sequence's block table sits in LDS so
// that a tile costs one memory round trip, not two), and every wave multiplies the same
// tile, in two steps of 32 keys, with its own NQT column tiles of 16 queries.  A column tile is (position block, head): with
// four heads per kv head a wave holds the same 16 positions of the four heads, so a K/V
// tile is fetched from memory once per kv head, not once per query head, and every 16-byte
// LDS read feeds NQT matrix instructions.
//
// The arithmetic is that of the decode kernel (attention_mfma.hip): S^T = K . Q^T with
// v_mfma_f32_16x16x32_bf16 so that a query's scores lie in the lanes of its column, softmax
// in float32 (exp2, log2(e) folded into the scale), P^T rounded to bfloat16 feeds
// O^T += V^T . P^T straight from registers.  Row m of the two K tiles of a step is key
// 8*(m/4) + m%4 (+4 for the second), which makes lane group j hold keys 8j..8j+7 of both
// products.  The accumulators are rescaled only when some running maximum moved.
//
// LDS rows are padded by 16 bytes: the 16 lanes that read one matrix operand together
// then fall into 16 different 16-byte bank groups.
//
// Reference: PagedAttention::forward prefill branch,
// /root/reference/src/models/layers/attention.rs:947-958 (varlen over cu_seqlens with a
// cached prefix); golden formula /root/reference/tests/probes/compare_flashinfer_probe.py:51-73.
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr float kLog2eP = 1.4426950408889634f;
constexpr int kKeys = 64;    // keys per tile (two steps of 32)
constexpr int kVPad = 8;     // bf16 elements of padding per LDS row
constexpr float kSlack = 8.f;  // how far (log2) a score may exceed the softmax reference point

__device__ __forceinline__ bf16x8 ld8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ void st8(bf16* p, bf16x8 v) { *reinterpret_cast<bf16x8*>(p) = v; }
__device__ __forceinline__ bf16x8 zero8p() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// NWV waves of NQT column tiles each: the workgroup's NWV * NQT tiles are (position block,
// head) pairs, GH heads per position block.  Eight waves of two tiles keep a wave within
// half of a SIMD's registers, so two waves share a SIMD and one's exponentials overlap the
// other's matrix instructions.
// FULLD: head_dim is exactly 16 * DT, so no row tile of V^T lies past the end and the
// products with V^T are straight-line code.
template <int KC, int DT, int NQT, int GH, int NWV, bool FULLD>
__global__ __launch_bounds__(64 * NWV, 2) void attn_prefill_lds_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ k_cache, const bf16* __restrict__ vt_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tiles,
    const int* __restrict__ cu_q, const int* __restrict__ ctx_lens, bf16* __restrict__ out, float scale_log2,
    int window, int page_shift, int nq, int nkv, int d) {
  const int page = 1 << page_shift;
  constexpr int NT = 64 * NWV;                    // threads
  constexpr int QB = 16 * (NWV * NQT / GH);       // query positions per workgroup
  constexpr int LI = (256 * KC + NT - 1) / NT;    // 16-byte chunks per thread and tile, for K and for V^T
  static_assert((NWV * NQT) % GH == 0, "tiles must divide into whole position blocks");
  extern __shared__ __align__(16) unsigned char smem[];
  constexpr int krow = 32 * KC + kVPad;  // elements per K row in LDS: head_dim rounded up to the
                                         // 32-wide steps of the matrix product (the rest is zero)
  const int vrow = kKeys + kVPad;       // elements per V^T row in LDS
  const int stage = kKeys * krow + d * vrow;
  bf16* lds = reinterpret_cast<bf16*>(smem);
  int* bt_s = reinterpret_cast<int*>(smem + 2 * (size_t)stage * sizeof(bf16));  // [max_pages]

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int g = nq / nkv, groups = g / GH;
  const int kvh = blockIdx.x / groups;
  const int h0 = kvh * g + (blockIdx.x - kvh * groups) * GH;
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
    const bf16* qrow = q + ((size_t)(q_begin + (ok ? qi : 0)) * nq + h0 + hh) * d;
#pragma unroll
    for (int c = 0; c < KC; ++c) {
      const int off = 32 * c + 8 * j;
      qb[ct][c] = (ok && off < d) ? ld8(qrow + off) : zero8p();
    }
    m_run[ct] = -INFINITY;
    l_run[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[dt][ct] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // ---- cooperative tile copy.  K tile: 64 keys of 4*KC 16-byte chunks (chunks past
  // head_dim are zero), thread t moves chunks t, t + 256, ...; in LDS the keys of each
  // 32-key step are permuted so that the 16 rows one matrix operand reads are consecutive:
  // key k sits at row 16*((k>>2)&1) + 4*(k>>3) + (k&3) of its step.  V^T tile: d rows of 8
  // key groups; thread t moves row t % d of key group t / d, .. (the pool keeps a key group's rows
  // side by side: threads that follow each other read 16 bytes that follow each other).
  constexpr int CPK = 4 * KC;        // chunks per K row in LDS
  const int n_vchunks = 8 * d;
  int c_kl[LI], c_koff[LI], c_kdst[LI], c_vdst[LI], c_vrow[LI], c_vkg[LI];
#pragma unroll
  for (int i = 0; i < LI; ++i) {
    const int idx = tid + NT * i;
    const int kl = idx / CPK, ch = idx % CPK;
    const int k32 = kl & 31;
    c_kl[i] = kl;
    c_koff[i] = 8 * ch < d ? 8 * ch : -1;       // -1: a chunk of zeros
    c_kdst[i] = ((kl & 32) + 16 * ((k32 >> 2) & 1) + 4 * (k32 >> 3) + (k32 & 3)) * krow + 8 * ch;
    c_vkg[i] = idx / d;
    c_vrow[i] = idx - c_vkg[i] * d;
    if (c_vkg[i] > 7) { c_vkg[i] = 7; c_vrow[i] = d - 1; }      // past the tile: read again what the last chunk reads, store nothing
    c_vdst[i] = c_vrow[i] * vrow + 8 * c_vkg[i];
  }
  const size_t kv_head_stride = (size_t)d << page_shift;     // elements of one (page, kv head) block
  bf16x8 kreg[LI], vreg[LI];
  auto fetch = [&](int kb) {
#pragma unroll
    for (int i = 0; i < LI; ++i) {
      int key = kb + c_kl[i];
      key = key > k_last ? k_last : key;
      const int kp = bt_s[key >> page_shift];
      const bf16* ksrc = k_cache + ((size_t)kp * nkv + kvh) * kv_head_stride +
                         (size_t)(key & (page - 1)) * d + (c_koff[i] < 0 ? 0 : c_koff[i]);
      kreg[i] = ld8(ksrc);
      int key0 = kb + 8 * c_vkg[i];
      key0 = key0 > k_last ? (k_last & ~7) : key0;
      const int vp = bt_s[key0 >> page_shift];
      vreg[i] = ld8(vt_cache + ((size_t)vp * nkv + kvh) * kv_head_stride +
                    ((size_t)((key0 & (page - 1)) >> 3) * d + c_vrow[i]) * 8);     // [offset / 8, d, 8]
    }
  };
  auto stash = [&](int buf) {
    bf16* Ks = lds + buf * stage;
    bf16* Vs = Ks + kKeys * krow;
#pragma unroll
    for (int i = 0; i < LI; ++i) {
      st8(Ks + c_kdst[i], c_koff[i] < 0 ? zero8p() : kreg[i]);   // zeroed here, not at the load: the
                                                                  // load stays in flight meanwhile
      if (tid + NT * i < n_vchunks) st8(Vs + c_vdst[i], vreg[i]);
    }
  };

  __syncthreads();   // the block table is in LDS
  fetch(k_begin);
  stash(0);
  // every load so far (the queries among them) has landed before the loop starts, so that
  // inside it only the tile in flight is ever waited for: vmcnt(0), other counters untouched
  __builtin_amdgcn_s_waitcnt(0x0F70);
  __syncthreads();
  int buf = 0;
  for (int kt = k_begin; kt <= wg_last; kt += kKeys) {
    const bool more = kt + kKeys <= wg_last;
    if (more) fetch(kt + kKeys);
#pragma unroll
    for (int sub = 0; sub < kKeys / 32; ++sub) {
    const int kb = kt + 32 * sub;
    if (active && kb >= wave_k_begin && kb <= last_pos) {
      const bf16* Ks = lds + buf * stage + 32 * sub * krow;
      const bf16* Vs = lds + buf * stage + kKeys * krow + 32 * sub;
      // a step needs the mask unless every key is at or before every query and inside every window
      const bool masked = (kb + 31 > first_pos) || (kb < lo_last);
      bf16x8 ka[2][KC];
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const int off = 32 * c + 8 * j;
        ka[0][c] = ld8(Ks + r * krow + off);
        ka[1][c] = ld8(Ks + (16 + r) * krow + off);
      }
      // ---- all scores of the step first: 2 * KC * NQT matrix instructions with nothing
      // between them that waits for their results
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
      // ---- this lane's largest score per column tile (raw: the scale is positive and is
      // applied with the shift).  The reference point m_run of the exponentials only has to
      // be near the maximum: it moves when some score exceeds it by more than 2^kSlack, which
      // is rare after the first keys; then the sums so far are rescaled.  P stays below
      // 2^kSlack.  One test for all column tiles keeps the common path free of branches.
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
        if (FULLD || 16 * dt < d) {
          const bf16x8 va = ld8(Vs + (16 * dt + r) * vrow + 8 * j);
#pragma unroll
          for (int ct = 0; ct < NQT; ++ct)
            acc[dt][ct] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb_[ct], acc[dt][ct], 0, 0, 0);
        }
      }
    }
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
    buf ^= 1;
  }

  if (!active) return;
#pragma unroll
  for (int ct = 0; ct < NQT; ++ct) {
    float lt = l_run[ct] + lane_xor<16>(l_run[ct]);
    lt += lane_xor<32>(lt);
    const int tile = wave * NQT + ct;
    const int pb = tile / GH, hh = tile - pb * GH;
    const int qi = q0_blk + 16 * pb + r;
    if (qi >= q_len) continue;
    const float inv = 1.f / lt;
    bf16* o = out + ((size_t)(q_begin + qi) * nq + h0 + hh) * d;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      if (16 * dt >= d) break;
      bf16* op = o + 16 * dt + 4 * j;
      const f32x4 a = acc[dt][ct];
      op[0] = __float2bfloat16(a[0] * inv);
      op[1] = __float2bfloat16(a[1] * inv);
      op[2] = __float2bfloat16(a[2] * inv);
      op[3] = __float2bfloat16(a[3] * inv);
    }
  }
}

// Column tiles of a workgroup by head size and shape: eight waves of two tiles up to 128, of
// one tile above (the accumulators of a tile take twice the registers there).  The small
// shape has four waves: half the query positions per workgroup, twice the workgroups, two
// of them resident on a compute unit.  It serves batches with too few query blocks to give
// every compute unit two workgroups of different length.
static inline int tiles_of(int d, int small) { return (d <= 128 ? 16 : 8) / (small ? 2 : 1); }
// Query heads of a kv head that one workgroup takes together.
static inline int heads_together(int g) { return g % 4 == 0 ? 4 : (g % 2 == 0 ? 2 : 1); }

}  // namespace xi

using namespace xi;

extern "C" {

int xi_attention_mfma_supported(int nq, int nkv, int d, int page);

// Query positions per workgroup for a head size and a number of query heads per kv head
// (the host builds `tiles` in steps of it).
int xi_attention_prefill_block(int d, int g, int small) { return 16 * (tiles_of(d, small) / heads_together(g)); }

// tiles int32 [n_tiles, 2] = (sequence, first query position of the block within the
// sequence's portion), first positions being multiples of xi_attention_prefill_block(d, g, small).
int xi_attention_prefill_bf16(const void* q, const void* k_cache, const void* vt_cache, const int* block_tables,
                              int max_pages, const int* tiles, int n_tiles, const int* cu_q,
                              const int* ctx_lens, void* out, float scale, int window, int page, int nq,
                              int nkv, int d, int small, hipStream_t stream) {
  XI_CHECK(xi_attention_mfma_supported(nq, nkv, d, page), "attention_prefill: unsupported sizes nq=%d nkv=%d d=%d page=%d",
           nq, nkv, d, page);
  XI_CHECK(n_tiles >= 0 && n_tiles <= 65535, "attention_prefill: %d query blocks are too many for one launch", n_tiles);
  if (n_tiles == 0) return 0;
  const int g = nq / nkv;
  const int gh = heads_together(g);
  dim3 grid(nkv * (g / gh), n_tiles);
  const float sl = scale * kLog2eP;
  XI_CHECK(sl > 0.f, "attention_prefill: the scale must be positive");
  int page_shift = -1;
  for (int b = 0; b < 31; ++b)
    if ((1 << b) == page) page_shift = b;
  XI_CHECK(page_shift >= 3, "attention_prefill: the page size %d must be a power of two of at least 8", page);
#define XI_PF(KC, DT, NQT, GH, NWV)                                                                     \
  do {                                                                                                  \
    auto kern = d == 16 * DT ? attn_prefill_lds_kernel<KC, DT, NQT, GH, NWV, true>                      \
                             : attn_prefill_lds_kernel<KC, DT, NQT, GH, NWV, false>;                    \
    const size_t lds = 2 * (size_t)(kKeys * (32 * KC + kVPad) + d * (kKeys + kVPad)) * sizeof(bf16) +   \
                       (size_t)max_pages * sizeof(int);                                                 \
    XI_CHECK(lds <= 160 * 1024, "attention_prefill: block tables of %d pages do not fit in LDS", max_pages); \
    if (lds > 48 * 1024) {                                                                              \
      hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, \
                                         (int)lds);                                                     \
      XI_CHECK(e == hipSuccess, "attention_prefill: cannot get %zu bytes of LDS: %s", lds,              \
               hipGetErrorString(e));                                                                   \
    }                                                                                                   \
    kern<<<grid, 64 * NWV, lds, stream>>>((const bf16*)q, (const bf16*)k_cache, (const bf16*)vt_cache,  \
                                          block_tables, max_pages, tiles, cu_q, ctx_lens, (bf16*)out,   \
                                          sl, window, page_shift, nq, nkv, d);                          \
  } while (0)
#define XI_PF_GH(KC, DT, NQT, NWV)             \
  do {                                         \
    if (gh == 4) XI_PF(KC, DT, NQT, 4, NWV);   \
    else if (gh == 2) XI_PF(KC, DT, NQT, 2, NWV); \
    else XI_PF(KC, DT, NQT, 1, NWV);           \
  } while (0)
  if (small) {
    if (d <= 64) XI_PF_GH(2, 4, 2, 4);
    else if (d <= 128) XI_PF_GH(4, 8, 2, 4);
    else XI_PF_GH(8, 16, 1, 4);
  } else {
    if (d <= 64) XI_PF_GH(2, 4, 2, 8);
    else if (d <= 128) XI_PF_GH(4, 8, 2, 8);
    else XI_PF_GH(8, 16, 1, 8);
  }
#undef XI_PF_GH
#undef XI_PF
  XI_LAUNCH_CHECK("attention_prefill");
  return 0;
}

}  // extern "C"
