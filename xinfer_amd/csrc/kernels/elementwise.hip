// Bandwidth-bound kernels: embedding gather, fused residual-add + RMSNorm,
// fused per-head q/k RMSNorm + rotary embedding + paged KV write, SiLU*mul.
// All reductions are float32 in an order fixed by the row alone, so a row's
// result does not depend on what else is in the batch.
#include "common.h"
#include "qk_row.h"

#include <algorithm>
#include <stdarg.h>
#include <stdio.h>

namespace xi {

static thread_local char g_error[512] = "";
void set_error(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
}

// ---------------------------------------------------------------------------------
// Embedding: out[t, :] = float(table[ids[t], :]) * scale         (reference call site:
// /root/reference/src/models/qwen3.rs:303, candle Embedding::forward; Qwen3 has no scale: 1)
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                             float* __restrict__ out, int H, float scale) {
  const int t = blockIdx.x;
  const T* row = table + (size_t)ids[t] * H;
  float* o = out + (size_t)t * H;
  if (scale == 1.0f) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_float(row[i]);
  } else {
    for (int i = threadIdx.x; i < H; i += blockDim.x) o[i] = to_float(row[i]) * scale;
  }
}

// Reads `n16` 16-byte words and keeps nothing: the read-only stream against which the
// weight-streaming kernels are measured (bench.py --peaks).  A workgroup takes whole chunks of
// `chunk16` words (consecutive addresses stay with one compute unit, as the rows of a weight do in
// the products); a wave reads 1 KB an instruction and keeps eight of them in flight.
__global__ __launch_bounds__(512) void stream_read_kernel(const uint4* __restrict__ p, size_t n16, size_t chunk16,
                                                          unsigned* __restrict__ sink) {
  unsigned acc = 0;
  const size_t chunks = (n16 + chunk16 - 1) / chunk16;
  for (size_t c = blockIdx.x; c < chunks; c += gridDim.x) {
    const size_t lo = c * chunk16, hi = lo + chunk16 < n16 ? lo + chunk16 : n16;
    size_t i = lo + threadIdx.x;
    for (; i + 7 * 512 < hi; i += 8 * 512) {
      uint4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = p[i + u * 512];
#pragma unroll
      for (int u = 0; u < 8; ++u) acc ^= v[u].x ^ v[u].y ^ v[u].z ^ v[u].w;
    }
    for (; i < hi; i += 512) {
      const uint4 v = p[i];
      acc ^= v.x ^ v.y ^ v.z ^ v.w;
    }
  }
  if (acc == 0x9e3779b9u && sink != nullptr) *sink = acc;      // keeps the loads alive; `sink` is null in use
}

// Soft cap of logits in place: x = cap * tanh(x / cap), in float32.
__global__ void softcap_kernel(float* __restrict__ x, size_t n, float cap) {
  const float inv = 1.0f / cap;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x)
    x[i] = cap * tanhf(x[i] * inv);
}

// ---------------------------------------------------------------------------------
// Fused residual add + RMSNorm (reference: attention_rs::norm::add_rms_norm at
// /root/reference/src/models/layers/others.rs:118-123; plain rms_norm at :83).
//   s = resid[row] (+ y[row]);  if rows == null the sum is written back to resid;
//   out[r] = s * rsqrt(mean(s^2) + eps) * w, rounded once to the output type.
// The residual stream is float32 in both precisions.
// ---------------------------------------------------------------------------------
// y may hold `parts` partial sums [parts, T, H] (part stride T*H elements), added in order.
template <typename TY, typename TO, int NT>
__global__ void add_rmsnorm_kernel(float* __restrict__ resid, const TY* __restrict__ y, int parts, size_t part_stride,
                                   const float* __restrict__ w, float eps, TO* __restrict__ out,
                                   const int* __restrict__ rows, int H) {
  __shared__ float scratch[NT / kWave];
  const int r = blockIdx.x;
  const int row = rows ? rows[r] : r;
  float* x = resid + (size_t)row * H;
  const TY* yr = y ? y + (size_t)row * H : nullptr;
  TO* o = out + (size_t)r * H;
  float ss = 0.f;
  // first pass: sum (written back or kept in the output buffer's place is not possible for
  // a narrower TO, so the sum is recomputed in the second pass from the same operands).
  for (int i = threadIdx.x; i < H; i += NT) {
    float s = x[i];
    if (yr)
      for (int p = 0; p < parts; ++p) s += to_float(yr[p * part_stride + i]);
    ss += s * s;
  }
  const float total = block_sum<NT / kWave>(ss, scratch);
  const float inv = rsqrtf(total / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += NT) {
    float s = x[i];
    if (yr) {
      for (int p = 0; p < parts; ++p) s += to_float(yr[p * part_stride + i]);
      if (!rows) x[i] = s;
    }
    o[i] = from_float<TO>(s * inv * w[i]);
  }
}

// The same, for widths that are a multiple of 4 up to 4 * NT * MAXV: every thread keeps its
// part of the row in registers, so the row is read once and all loads are in flight
// together (one row of a decode step is otherwise a chain of dependent memory round trips).
struct alignas(8) bf16x4_t { bf16 v[4]; };
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16* p) {
  const bf16x4_t t = *reinterpret_cast<const bf16x4_t*>(p);
  return float4{to_float(t.v[0]), to_float(t.v[1]), to_float(t.v[2]), to_float(t.v[3])};
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16* p, float4 v) {
  bf16x4_t t;
  t.v[0] = from_float<bf16>(v.x);
  t.v[1] = from_float<bf16>(v.y);
  t.v[2] = from_float<bf16>(v.z);
  t.v[3] = from_float<bf16>(v.w);
  *reinterpret_cast<bf16x4_t*>(p) = t;
}

// PB: parts of a stack of partial sums whose loads are issued together (the sums run in order).
template <typename TY, typename TO, int NT, int MAXV, int PB>
__global__ __launch_bounds__(NT) void add_rmsnorm_vec_kernel(float* __restrict__ resid, const TY* __restrict__ y,
                                                             int parts, size_t part_stride,
                                                             const float* __restrict__ w, float eps,
                                                             TO* __restrict__ out, const int* __restrict__ rows,
                                                             int H) {
  __shared__ float scratch[NT / kWave];
  const int r = blockIdx.x;
  const int row = rows ? rows[r] : r;
  float* x = resid + (size_t)row * H;
  const TY* yr = y ? y + (size_t)row * H : nullptr;
  TO* o = out + (size_t)r * H;
  const int nvec = H / 4;
  float4 s[MAXV], wv[MAXV];
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = v * NT + threadIdx.x;
    if (i < nvec) {
      s[v] = load4(x + 4 * i);
      wv[v] = load4(w + 4 * i);
      if (yr) {
        // up to PB parts at a time: their loads are issued together, the sums run in order
        for (int p0 = 0; p0 < parts; p0 += PB) {
          float4 yy[PB];
#pragma unroll
          for (int p = 0; p < PB; ++p)
            yy[p] = p0 + p < parts ? load4(yr + (p0 + p) * part_stride + 4 * i) : float4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int p = 0; p < PB; ++p)
            if (p0 + p < parts) {
              s[v].x += yy[p].x;
              s[v].y += yy[p].y;
              s[v].z += yy[p].z;
              s[v].w += yy[p].w;
            }
        }
      }
    } else {
      s[v] = float4{0.f, 0.f, 0.f, 0.f};
      wv[v] = s[v];
    }
  }
  float ss = 0.f;
#pragma unroll
  for (int v = 0; v < MAXV; ++v) ss += (s[v].x * s[v].x + s[v].y * s[v].y) + (s[v].z * s[v].z + s[v].w * s[v].w);
  const float total = block_sum<NT / kWave>(ss, scratch);
  const float inv = rsqrtf(total / (float)H + eps);
#pragma unroll
  for (int v = 0; v < MAXV; ++v) {
    const int i = v * NT + threadIdx.x;
    if (i < nvec) {
      if (yr && !rows) store4(x + 4 * i, s[v]);
      store4(o + 4 * i, float4{s[v].x * inv * wv[v].x, s[v].y * inv * wv[v].y, s[v].z * inv * wv[v].z,
                               s[v].w * inv * wv[v].w});
    }
  }
}

// ---------------------------------------------------------------------------------
// SiLU(gate) * up on a packed [T, 2I] buffer (reference: attention_rs::silu_and_mul at
// /root/reference/src/models/layers/mlp.rs:627-628; golden formula
// /root/reference/tests/probes/compare_attention_misc_probe.py:81-86).
// ---------------------------------------------------------------------------------
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ gu, T* __restrict__ out, int I, size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = to_float(gu[t * 2 * I + i]);
    const float u = to_float(gu[t * 2 * I + I + i]);
    const float s = g / (1.f + __expf(-g));
    out[idx] = from_float<T>(s * u);
  }
}
template <>
__global__ void silu_mul_kernel<float>(const float* __restrict__ gu, float* __restrict__ out, int I,
                                       size_t total) {
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total; idx += stride) {
    const size_t t = idx / I;
    const int i = (int)(idx - t * I);
    const float g = gu[t * 2 * I + i];
    const float u = gu[t * 2 * I + I + i];
    const float s = g / (1.f + expf(-g));  // full-precision exp on the 32-bit path
    out[idx] = s * u;
  }
}

// bfloat16 with I a multiple of 8: 16-byte loads and stores.
struct alignas(16) bf16x8_t { bf16 v[8]; };
__global__ void silu_mul_vec8_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int I, size_t total8) {
  const int per_row = I / 8;
  size_t idx = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; idx < total8; idx += stride) {
    const size_t t = idx / per_row;
    const int c = (int)(idx - t * per_row);
    const bf16x8_t g = *reinterpret_cast<const bf16x8_t*>(gu + t * 2 * I + 8 * c);
    const bf16x8_t u = *reinterpret_cast<const bf16x8_t*>(gu + t * 2 * I + I + 8 * c);
    bf16x8_t o;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float gf = to_float(g.v[e]);
      o.v[e] = from_float<bf16>(gf / (1.f + __expf(-gf)) * to_float(u.v[e]));
    }
    *reinterpret_cast<bf16x8_t*>(out + t * I + 8 * c) = o;
  }
}

// ---------------------------------------------------------------------------------
// Per-head q/k RMSNorm + rotary embedding + KV write into the paged cache.
// One wave per (token, head) over the packed projection row [q heads | k heads | v heads].
//   q, k: x = rms(x, w) if w given (reference attention.rs:734-741); then the first
//   `rot` dims are rotated by the token's position (rotary_emb.rs:103; formula
//   tests/probes/compare_attention_misc_probe.py:33-49):
//     half layout:        pairs (i, i + rot/2);   interleaved layout: pairs (2i, 2i+1)
//     o_a = a*cos - b*sin;  o_b = a*sin + b*cos
//   q goes to q_out [T, nq, d]; k and v go to cache[page, kv_head, offset, :] with
//   slot = page*page_size + offset (reference slot formula runner.rs:1344-1362); with
//   v_grouped the V pool is [page, kv_head, offset / 8, d, 8]: eight keys that follow each other lie
//   side by side for every dim (the 16 bytes a lane of the MFMA attention reads), and a token's d
//   values fall into d / 8 lines of 128 bytes (into d lines if a whole page's keys lay side by side).
//   A negative slot means: do not store (the token's cache belongs to another run).
//   `bias` (float32, one value per element of the packed row, or null) is the projections'
//   bias: it is added here, in float32, to the product the row holds (q, k and v alike;
//   reference attention.rs:819-828 adds it in the linear layer).
// ---------------------------------------------------------------------------------
// PARTS: the packed rows come as `slices` float32 partial sums [slices, T, heads * d] (a product
// cut along K, `slice_stride` elements apart), added here in slice order.
template <typename T, bool PARTS>
__global__ void qk_norm_rope_kv_kernel(const void* __restrict__ qkv_v, int slices, size_t slice_stride,
                                       const float* __restrict__ bias,
                                       const float* __restrict__ qw,
                                       const float* __restrict__ kw, float eps,
                                       const float* __restrict__ cos_t,
                                       const float* __restrict__ sin_t, int rot, int interleaved,
                                       const int* __restrict__ positions,
                                       const long long* __restrict__ slots, T* __restrict__ q_out,
                                       T* __restrict__ k_cache, T* __restrict__ v_cache,
                                       int page_size, int n_tok, int nq, int nkv, int d, int v_grouped) {
  const int heads = nq + 2 * nkv;
  const int lane = threadIdx.x & (kWave - 1);
  const long long wid = (long long)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
  if (wid >= (long long)n_tok * heads) return;
  const int t = (int)(wid / heads);
  const int h = (int)(wid - (long long)t * heads);
  const PackedHead<T, PARTS> x{qkv_v, (size_t)t * heads * d + (size_t)h * d, slices, slice_stride,
                               bias ? bias + (size_t)h * d : nullptr};
  if (h < nq) {
    norm_rope_head<T, PARTS>(x, qw, eps, cos_t, sin_t, rot, interleaved, positions[t], d, lane,
                             q_out + ((size_t)t * nq + h) * d);
    return;
  }
  const long long slot = slots[t];
  if (slot < 0) return;
  const long long page = slot / page_size;
  const int off = (int)(slot - page * page_size);
  const bool is_k = h < nq + nkv;
  const int kvh = is_k ? h - nq : h - nq - nkv;
  if (is_k)
    norm_rope_head<T, PARTS>(x, kw, eps, cos_t, sin_t, rot, interleaved, positions[t], d, lane,
                             k_cache + (((size_t)page * nkv + kvh) * page_size + off) * d);
  else if (v_grouped)      // V kept as [page, kv_head, offset / 8, d, 8]
    copy_head<T, PARTS>(x, d, lane, v_cache + ((size_t)page * nkv + kvh) * d * page_size + (size_t)(off >> 3) * d * 8 + (off & 7),
                        (size_t)8);
  else
    copy_head<T, PARTS>(x, d, lane, v_cache + (((size_t)page * nkv + kvh) * page_size + off) * d, 1);
}

// The same for bfloat16 with the V pool in groups of eight keys, 16 bytes per lane and one pass: a
// workgroup owns one head of the packed row for a block of consecutive tokens.  A head of a
// token is d/8 lanes of 8 elements (sums and the rotary partner are exchanged inside that
// group of lanes), a wave holds 64/(d/8) tokens, the workgroup's waves hold the block.  The
// workgroup of a V head turns its [tokens, d] tile through LDS so that a wave's store takes eight
// tokens by eight dims: where the eight tokens follow each other in a group of the pool, one line
// of 128 bytes.
// Needs d % 8 == 0 and, for the half layout, rotary_dim % 16 == 0 (the partner of a lane's
// 8 elements is then another lane's 8 elements).
struct alignas(16) bf16x8v { bf16 v[8]; };

__global__ __launch_bounds__(1024) void qk_norm_rope_kvt_bf16_kernel(
    const bf16* __restrict__ qkv, const float* __restrict__ bias, const float* __restrict__ qw, const float* __restrict__ kw, float eps,
    const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot, int interleaved,
    const int* __restrict__ positions, const long long* __restrict__ slots, bf16* __restrict__ q_out,
    bf16* __restrict__ k_cache, bf16* __restrict__ vt_cache, int page_size, int n_tok, int nq, int nkv, int d) {
  extern __shared__ __align__(16) unsigned char smem_raw[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int heads = nq + 2 * nkv;
  const int lph = d >> 3;          // lanes per head
  const int hpw = 64 / lph;        // tokens a wave holds
  const int tpw = (blockDim.x >> 6) * hpw;   // tokens of the workgroup (at most 64)
  const int sub = lane / lph, c = lane - sub * lph;
  const int h = blockIdx.y;
  const int t0 = blockIdx.x * tpw;
  const int tl = wave * hpw + sub;  // this lane's token within the block
  const int t = t0 + tl;
  const bool on = sub < hpw && t < n_tok;

  if (h >= nq + nkv) {
    // ---- a V head: tile into LDS, then lanes along the token axis
    const int kvh = h - nq - nkv;
    bf16* vs = reinterpret_cast<bf16*>(smem_raw);  // [tpw][d + 2]
    const int vstride = d + 2;                      // an odd number of 32-bit words per row
    // Every lane looks up where its own token of the block goes (lane = token); a store then takes eight
    // tokens by eight dims: lane -> token 8 tg + (lane & 7), dim i0 + (lane >> 3), the place handed over
    // from the token's lane.
    const long long slot = (lane < tpw && t0 + lane < n_tok) ? slots[t0 + lane] : -1;
    unsigned long long place = ~0ull;          // of the token's dim 0 in the pool, in elements
    if (slot >= 0) {
      const long long page = slot / page_size;
      const int off = (int)(slot - page * page_size);
      place = ((unsigned long long)page * nkv + kvh) * d * page_size + (unsigned long long)(off >> 3) * d * 8 + (off & 7);
    }
    if (on) {
      uint4 raw = *reinterpret_cast<const uint4*>(qkv + ((size_t)t * heads + h) * d + 8 * c);
      if (bias) {
        bf16x8v x = *reinterpret_cast<const bf16x8v*>(&raw);
#pragma unroll
        for (int e = 0; e < 8; ++e) x.v[e] = from_float<bf16>(to_float(x.v[e]) + bias[(size_t)h * d + 8 * c + e]);
        raw = *reinterpret_cast<const uint4*>(&x);
      }
      unsigned* dst = reinterpret_cast<unsigned*>(vs + tl * vstride + 8 * c);
      dst[0] = raw.x;
      dst[1] = raw.y;
      dst[2] = raw.z;
      dst[3] = raw.w;
    }
    __syncthreads();
    const int units = ((tpw + 7) >> 3) * (d >> 3);
    for (int u = wave; u < units; u += (int)(blockDim.x >> 6)) {
      const int tg = u / (d >> 3), i = 8 * (u - tg * (d >> 3)) + (lane >> 3);
      const int tok = 8 * tg + (lane & 7);
      const unsigned lo = __shfl((unsigned)place, tok, kWave), hi = __shfl((unsigned)(place >> 32), tok, kWave);
      const unsigned long long at = ((unsigned long long)hi << 32) | lo;
      if (at != ~0ull) vt_cache[at + (size_t)i * 8] = vs[tok * vstride + i];
    }
    return;
  }

  // ---- a query head or a k head
  const bool is_k = h >= nq;
  float v[8];
  {
    bf16x8v x;
    if (on) x = *reinterpret_cast<const bf16x8v*>(qkv + ((size_t)t * heads + h) * d + 8 * c);
#pragma unroll
    for (int e = 0; e < 8; ++e) v[e] = on ? to_float(x.v[e]) + (bias ? bias[(size_t)h * d + 8 * c + e] : 0.f) : 0.f;
  }
  const float* w = is_k ? kw : qw;
  if (w) {
    float ss = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) ss += v[e] * v[e];
    float total;
    if ((lph & (lph - 1)) == 0) {
      total = ss;
      for (int off = 1; off < lph; off <<= 1) total += __shfl_xor(total, off, kWave);
    } else {
      total = 0.f;
      const int first = lane - c;
      for (int o = 0; o < lph; ++o) total += __shfl(ss, first + o, kWave);
    }
    const float inv = rsqrtf(total / (float)d + eps);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      v[e] *= inv;
      v[e] *= w[8 * c + e];
    }
  }
  const int half = rot >> 1;
  const int pos = positions[t < n_tok ? t : n_tok - 1];
  float o[8];
  if (interleaved) {
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      const int i = 8 * c + e;
      if (i < rot) {
        const float cs = cos_t[(size_t)pos * half + (i >> 1)], sn = sin_t[(size_t)pos * half + (i >> 1)];
        o[e] = v[e] * cs - v[e + 1] * sn;
        o[e + 1] = v[e] * sn + v[e + 1] * cs;
      } else {
        o[e] = v[e];
        o[e + 1] = v[e + 1];
      }
    }
  } else {
    const int hop = rot >> 4;        // lanes between rotary partners
    const bool in_rot = 8 * c < rot;
    const bool first = 8 * c < half;
    int partner = first ? lane + hop : lane - hop;
    if (!in_rot) partner = lane;
    const int p0 = first ? 8 * c : 8 * c - half;   // pair index of this lane's first element
    float cs[8], sn[8];
    if (in_rot) {
      const float4* cp = reinterpret_cast<const float4*>(cos_t + (size_t)pos * half + p0);
      const float4* sp = reinterpret_cast<const float4*>(sin_t + (size_t)pos * half + p0);
      const float4 c0 = cp[0], c1 = cp[1], s0 = sp[0], s1 = sp[1];
      cs[0] = c0.x; cs[1] = c0.y; cs[2] = c0.z; cs[3] = c0.w; cs[4] = c1.x; cs[5] = c1.y; cs[6] = c1.z; cs[7] = c1.w;
      sn[0] = s0.x; sn[1] = s0.y; sn[2] = s0.z; sn[3] = s0.w; sn[4] = s1.x; sn[5] = s1.y; sn[6] = s1.z; sn[7] = s1.w;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pv = __shfl(v[e], partner, kWave);
      o[e] = !in_rot ? v[e] : (first ? v[e] * cs[e] - pv * sn[e] : pv * sn[e] + v[e] * cs[e]);
    }
  }
  if (!on) return;
  bf16x8v y;
#pragma unroll
  for (int e = 0; e < 8; ++e) y.v[e] = from_float<bf16>(o[e]);
  if (!is_k) {
    *reinterpret_cast<bf16x8v*>(q_out + ((size_t)t * nq + h) * d + 8 * c) = y;
  } else {
    const long long slot = slots[t];
    if (slot >= 0) {
      const long long page = slot / page_size;
      const int off = (int)(slot - page * page_size);
      *reinterpret_cast<bf16x8v*>(k_cache + (((size_t)page * nkv + (h - nq)) * page_size + off) * d + 8 * c) = y;
    }
  }
}

// out[i][l] = in[l ^ (1 << i)] for i = 0 .. 5, by `lane_xor` (for its test)
__global__ void lane_xor_probe_kernel(const float* __restrict__ in, float* __restrict__ out) {
  const int l = threadIdx.x;
  const float v = in[l];
  out[0 * kWave + l] = lane_xor<1>(v);
  out[1 * kWave + l] = lane_xor<2>(v);
  out[2 * kWave + l] = lane_xor<4>(v);
  out[3 * kWave + l] = lane_xor<8>(v);
  out[4 * kWave + l] = lane_xor<16>(v);
  out[5 * kWave + l] = lane_xor<32>(v);
  out[6 * kWave + l] = wave_sum(v);
  out[7 * kWave + l] = wave_max(v);
}

}  // namespace xi

using namespace xi;

extern "C" {

const char* xi_last_error() { return g_error; }

// in [64] float32 -> out [8][64]: lanes exchanged across 1, 2, 4, 8, 16, 32, the wave's sum and maximum
int xi_lane_xor_probe(const float* in, float* out, hipStream_t stream) {
  lane_xor_probe_kernel<<<1, kWave, 0, stream>>>(in, out);
  XI_LAUNCH_CHECK("lane_xor_probe");
  return 0;
}

int xi_embed(const void* table, int dtype, const int* ids, float* out, int n_tok, int H, float scale,
             hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && H > 0, "embed: bad sizes T=%d H=%d", n_tok, H);
  if (n_tok == 0) return 0;
  if (dtype == kF32)
    embed_kernel<float><<<n_tok, 256, 0, stream>>>((const float*)table, ids, out, H, scale);
  else if (dtype == kBF16)
    embed_kernel<bf16><<<n_tok, 256, 0, stream>>>((const bf16*)table, ids, out, H, scale);
  else
    XI_CHECK(false, "embed: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("embed");
  return 0;
}

int xi_stream_read(const void* p, int64_t bytes, int workgroups, int64_t chunk_bytes, hipStream_t stream) {
  XI_CHECK(bytes >= 0 && workgroups > 0 && workgroups <= 65535 && chunk_bytes >= 8192 && chunk_bytes % 8192 == 0 &&
               ((uintptr_t)p & 15) == 0,
           "stream_read: bad arguments bytes=%lld workgroups=%d chunk=%lld", (long long)bytes, workgroups,
           (long long)chunk_bytes);
  if (bytes < 16) return 0;
  stream_read_kernel<<<workgroups, 512, 0, stream>>>((const uint4*)p, (size_t)(bytes / 16), (size_t)(chunk_bytes / 16),
                                                     nullptr);
  XI_LAUNCH_CHECK("stream_read");
  return 0;
}

int xi_softcap(float* x, int64_t n, float cap, hipStream_t stream) {
  XI_CHECK(n >= 0 && cap > 0.f, "softcap: bad sizes n=%lld cap=%g", (long long)n, (double)cap);
  if (n == 0) return 0;
  const int blocks = (int)std::min<int64_t>((n + 255) / 256, 4096);
  softcap_kernel<<<blocks, 256, 0, stream>>>(x, (size_t)n, cap);
  XI_LAUNCH_CHECK("softcap");
  return 0;
}

// y may be null (no add).  rows may be null (all n_rows rows in place).
// y: null, [T, H], or `parts` partial sums [parts, T, H] (T = resid_rows), added in order.
int xi_add_rmsnorm(float* resid, const void* y, int y_dtype, int parts, int resid_rows, const float* w, float eps,
                   void* out, int out_dtype, const int* rows, int n_rows, int H, hipStream_t stream) {
  XI_CHECK(n_rows >= 0 && H > 0, "add_rmsnorm: bad sizes rows=%d H=%d", n_rows, H);
  XI_CHECK(parts >= 1 && resid_rows >= 0, "add_rmsnorm: bad partial sums (%d parts of %d rows)", parts, resid_rows);
  const size_t part_stride = (size_t)resid_rows * H;
  if (n_rows == 0) return 0;
  constexpr int NT = 256, MAXV = 8;
  const bool vec = H % 4 == 0 && H <= 4 * NT * MAXV && ((uintptr_t)resid | (uintptr_t)y | (uintptr_t)w | (uintptr_t)out) % 16 == 0;
  // Few rows (a decode step, which may add a stack of partial sums of its o and down products):
  // with one workgroup a row the kernel lives on the latency of its chain of loads, so a row
  // gets 1024 threads and up to 8 parts are asked for at once.  The parts are added in the same
  // order.  Measured on MI355X, 64 rows of 4096 with 8 parts: 4.0 us against 8.6.
  const bool few = vec && n_rows <= 256 && H <= 4 * 1024 * 2;
#define XI_NORM(TY, TO)                                                                            \
  do {                                                                                             \
    if (few)                                                                                       \
      add_rmsnorm_vec_kernel<TY, TO, 1024, 2, 8><<<n_rows, 1024, 0, stream>>>(                     \
          resid, (const TY*)y, parts, part_stride, w, eps, (TO*)out, rows, H);                     \
    else if (vec)                                                                                  \
      add_rmsnorm_vec_kernel<TY, TO, NT, MAXV, 4><<<n_rows, NT, 0, stream>>>(                      \
          resid, (const TY*)y, parts, part_stride, w, eps, (TO*)out, rows, H);                     \
    else                                                                                           \
      add_rmsnorm_kernel<TY, TO, NT><<<n_rows, NT, 0, stream>>>(resid, (const TY*)y, parts,        \
                                                                part_stride, w, eps, (TO*)out,     \
                                                                rows, H);                          \
  } while (0)
  if (y_dtype == kF32 && out_dtype == kF32) XI_NORM(float, float);
  else if (y_dtype == kBF16 && out_dtype == kBF16) XI_NORM(bf16, bf16);
  else if (y_dtype == kF32 && out_dtype == kBF16) XI_NORM(float, bf16);
  else if (y_dtype == kBF16 && out_dtype == kF32) XI_NORM(bf16, float);
  else XI_CHECK(false, "add_rmsnorm: unknown dtypes %d %d", y_dtype, out_dtype);
#undef XI_NORM
  XI_LAUNCH_CHECK("add_rmsnorm");
  return 0;
}

int xi_silu_mul(const void* gate_up, void* out, int dtype, int n_tok, int I, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && I > 0, "silu_mul: bad sizes T=%d I=%d", n_tok, I);
  if (n_tok == 0) return 0;
  const size_t total = (size_t)n_tok * I;
  const int nt = 256;
  size_t blocks = (total + nt - 1) / nt;
  if (blocks > 65535u * 16u) blocks = 65535u * 16u;
  if (dtype == kF32)
    silu_mul_kernel<float><<<(unsigned)blocks, nt, 0, stream>>>((const float*)gate_up, (float*)out, I, total);
  else if (dtype == kBF16 && I % 8 == 0 && ((uintptr_t)gate_up | (uintptr_t)out) % 16 == 0) {
    const size_t total8 = total / 8;
    size_t b8 = (total8 + nt - 1) / nt;
    if (b8 > 65535u * 16u) b8 = 65535u * 16u;
    silu_mul_vec8_kernel<<<(unsigned)b8, nt, 0, stream>>>((const bf16*)gate_up, (bf16*)out, I, total8);
  } else if (dtype == kBF16)
    silu_mul_kernel<bf16><<<(unsigned)blocks, nt, 0, stream>>>((const bf16*)gate_up, (bf16*)out, I, total);
  else
    XI_CHECK(false, "silu_mul: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("silu_mul");
  return 0;
}

// qkv: [T, heads * d] in `dtype`, or, with slices > 0, float32 partial sums [slices, T, heads * d]
// of it (then `dtype` is that of q_out and the cache, and the form of one wave per head runs).
int xi_qk_norm_rope_kv(const void* qkv, int dtype, int slices, const float* bias, const float* qw, const float* kw, float eps,
                       const float* cos_t, const float* sin_t, int rot, int interleaved,
                       const int* positions, const long long* slots, void* q_out, void* k_cache,
                       void* v_cache, int page_size, int n_tok, int nq, int nkv, int d, int v_grouped,
                       int vector_min_tokens, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && nq > 0 && nkv > 0 && d > 0 && page_size > 0,
           "qk_norm_rope_kv: bad sizes T=%d nq=%d nkv=%d d=%d page=%d", n_tok, nq, nkv, d, page_size);
  XI_CHECK(rot >= 0 && rot <= d && rot % 2 == 0, "qk_norm_rope_kv: rotary_dim %d must be even and <= head_dim %d", rot, d);
  XI_CHECK(d <= 256, "qk_norm_rope_kv: head_dim %d exceeds 256", d);
  XI_CHECK((qw == nullptr) == (kw == nullptr), "qk_norm_rope_kv: q and k norm weights must both be given or both absent");
  if (n_tok == 0) return 0;
  // Many tokens (prompt portions): the vectorized form.  Few (decode steps): one wave per
  // (token, head) below, whose shorter chain of dependent loads finishes sooner.
  XI_CHECK(slices >= 0 && slices <= 64, "qk_norm_rope_kv: %d slices", slices);
  XI_CHECK(!v_grouped || page_size % 8 == 0, "qk_norm_rope_kv: V in groups of eight keys needs pages of a multiple of 8 tokens, not %d",
           page_size);
  if (slices == 0 && n_tok >= vector_min_tokens && dtype == kBF16 && v_grouped && d % 8 == 0 && d <= 256 &&
      (interleaved || rot % 16 == 0) &&
      ((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)k_cache | (uintptr_t)cos_t | (uintptr_t)sin_t) % 16 == 0) {
    const int lph = d / 8, hpw = 64 / lph;
    int n_waves = 64 / hpw;                       // waves of a workgroup: at most 64 tokens, at most 16 waves
    if (n_waves > 16) n_waves = 16;
    const int tpw = n_waves * hpw;
    const unsigned blocks_x = (unsigned)((n_tok + tpw - 1) / tpw);
    XI_CHECK(nq + 2 * nkv <= 65535, "qk_norm_rope_kv: too many heads");
    const size_t lds = (size_t)tpw * (d + 2) * sizeof(bf16);
    qk_norm_rope_kvt_bf16_kernel<<<dim3(blocks_x, nq + 2 * nkv), n_waves * 64, lds, stream>>>(
        (const bf16*)qkv, bias, qw, kw, eps, cos_t, sin_t, rot, interleaved, positions, slots, (bf16*)q_out,
        (bf16*)k_cache, (bf16*)v_cache, page_size, n_tok, nq, nkv, d);
    XI_LAUNCH_CHECK("qk_norm_rope_kv");
    return 0;
  }
  const long long waves = (long long)n_tok * (nq + 2 * nkv);
  const int wpb = 4;
  const long long blocks = (waves + wpb - 1) / wpb;
  XI_CHECK(blocks < (1ll << 31), "qk_norm_rope_kv: too many tokens");
  const size_t slice_stride = (size_t)n_tok * (nq + 2 * nkv) * d;
#define XI_QK(TT, PARTS)                                                                        \
  qk_norm_rope_kv_kernel<TT, PARTS><<<(unsigned)blocks, wpb * kWave, 0, stream>>>(              \
      qkv, slices, slice_stride, bias, qw, kw, eps, cos_t, sin_t, rot, interleaved, positions, slots, (TT*)q_out, \
      (TT*)k_cache, (TT*)v_cache, page_size, n_tok, nq, nkv, d, v_grouped)
  if (dtype == kF32 && slices == 0) XI_QK(float, false);
  else if (dtype == kF32) XI_QK(float, true);
  else if (dtype == kBF16 && slices == 0) XI_QK(bf16, false);
  else if (dtype == kBF16) XI_QK(bf16, true);
  else XI_CHECK(false, "qk_norm_rope_kv: unknown dtype %d", dtype);
#undef XI_QK
  XI_LAUNCH_CHECK("qk_norm_rope_kv");
  return 0;
}

}  // extern "C"
