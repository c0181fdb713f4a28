// One head of one token of a packed projection row, by one wave: the per-head RMSNorm and the
// rotation of a q or k head, and the copy of a v head.  Shared by the kernel that does this for a
// whole step and by the decode attention kernel that does it for its own heads, so that both
// give the same bits.
//   x = rms(x, w) if w is given (reference attention.rs:734-741); then the first `rot` dims
//   are rotated by the token's position (rotary_emb.rs:103; formula
//   tests/probes/compare_attention_misc_probe.py:33-49):
//     half layout:        pairs (i, i + rot/2);   interleaved layout: pairs (2i, 2i+1)
//     o_a = a*cos - b*sin;  o_b = a*sin + b*cos
#pragma once
#include "common.h"

namespace xi {

// Where a head's elements come from: a row of T, or (PARTS) `slices` float32 partial sums
// `slice_stride` elements apart (a product cut along K), added in slice order.
template <typename T, bool PARTS>
struct PackedHead {
  const void* base;      // the packed rows
  size_t row0;           // index of the head's first element
  int slices;
  size_t slice_stride;
  const float* bias;     // the head's bias (float32, added to the product), or null
  __device__ __forceinline__ float raw(int i) const {
    if constexpr (PARTS) {
      const float* p = reinterpret_cast<const float*>(base) + row0 + i;
      float a = 0.f;
#pragma unroll 4
      for (int sl = 0; sl < slices; ++sl) a += p[(size_t)sl * slice_stride];
      return a;
    } else {
      return to_float(reinterpret_cast<const T*>(base)[row0 + i]);
    }
  }
  __device__ __forceinline__ float at(int i) const { return bias ? raw(i) + bias[i] : raw(i); }
};

// v: element i goes to dst[i * stride], rounded once.
template <typename T, bool PARTS>
__device__ __forceinline__ void copy_head(const PackedHead<T, PARTS>& x, int d, int lane, T* dst, size_t stride) {
  for (int i = lane; i < d; i += kWave) dst[(size_t)i * stride] = from_float<T>(x.at(i));
}

// q or k: norm (if `w`), rotation, one rounding, to dst[0..d).  head_dim <= 256.
// In two steps, so that a caller can ask for everything first and use it after other work: `load`
// asks for the head's elements, the norm's weights and the position's row of the tables at once (a
// lane holds pairs lane and lane + 64 of the rotated part and up to 4 elements of the rest),
// `finish` norms, rotates and stores.
template <typename T, bool PARTS>
struct HeadRegs {
  float xa[2], xb[2], wa[2], wb[2], xt[4], wt[4], cs[2], sn[2];

  __device__ __forceinline__ void load(const PackedHead<T, PARTS>& x, const float* __restrict__ w,
                                       const float* __restrict__ cos_t, const float* __restrict__ sin_t, int rot,
                                       int interleaved, int pos, int d, int lane) {
    const int half = rot / 2;
    const float* bs = x.bias;
    // (a group of 64 lanes none of which holds anything is skipped as a whole: the tests on p are
    // the same for every lane)
    const float* c = cos_t + (size_t)pos * half;
    const float* sn_row = sin_t + (size_t)pos * half;
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      xa[p] = xb[p] = 0.f;
      wa[p] = wb[p] = 1.f;
      cs[p] = 1.f;
      sn[p] = 0.f;
      if (kWave * p >= half) continue;
      const int i = lane + kWave * p;
      const bool ok = i < half;
      const int ia = interleaved ? 2 * i : i;
      const int ib = interleaved ? 2 * i + 1 : i + half;
      xa[p] = ok ? x.raw(ia) + (bs ? bs[ia] : 0.f) : 0.f;
      xb[p] = ok ? x.raw(ib) + (bs ? bs[ib] : 0.f) : 0.f;
      wa[p] = (ok && w) ? w[ia] : 1.f;
      wb[p] = (ok && w) ? w[ib] : 1.f;
      cs[p] = ok ? c[i] : 1.f;
      sn[p] = ok ? sn_row[i] : 0.f;
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) {
      xt[p] = 0.f;
      wt[p] = 1.f;
      if (rot + kWave * p >= d) continue;
      const int i = rot + lane + kWave * p;
      const bool ok = i < d;
      xt[p] = ok ? x.raw(i) + (bs ? bs[i] : 0.f) : 0.f;
      wt[p] = (ok && w) ? w[i] : 1.f;
    }
  }

  // Every product and sum is written out (no contraction left to the compiler), so that the
  // result does not depend on the code around a call.
  __device__ __forceinline__ void finish(bool normed, float eps, int rot, int interleaved, int d, int lane, T* dst) const {
#pragma clang fp contract(off)
    const int half = rot / 2;
    float inv = 1.f;
    if (normed) {
      float ss = 0.f;
#pragma unroll
      for (int p = 0; p < 2; ++p) ss = __builtin_fmaf(xb[p], xb[p], __builtin_fmaf(xa[p], xa[p], ss));
#pragma unroll
      for (int p = 0; p < 4; ++p) ss = __builtin_fmaf(xt[p], xt[p], ss);
      ss = wave_sum(ss);
      inv = rsqrtf(ss / (float)d + eps);
    }
#pragma unroll
    for (int p = 0; p < 2; ++p) {
      if (kWave * p >= half) continue;
      const int i = lane + kWave * p;
      if (i < half) {
        // the reference rounds the normed value to the activation type before rotating
        // (two kernels); here it stays in float32 until the single final rounding.
        const float a = xa[p] * inv * wa[p];
        const float b = xb[p] * inv * wb[p];
        dst[interleaved ? 2 * i : i] = from_float<T>(__builtin_fmaf(a, cs[p], -(b * sn[p])));
        dst[interleaved ? 2 * i + 1 : i + half] = from_float<T>(__builtin_fmaf(a, sn[p], b * cs[p]));
      }
    }
#pragma unroll
    for (int p = 0; p < 4; ++p) {  // dims beyond the rotary part
      if (rot + kWave * p >= d) continue;
      const int i = rot + lane + kWave * p;
      if (i < d) dst[i] = from_float<T>(xt[p] * inv * wt[p]);
    }
  }
};

template <typename T, bool PARTS>
__device__ __forceinline__ void norm_rope_head(const PackedHead<T, PARTS>& x, const float* __restrict__ w, float eps,
                                               const float* __restrict__ cos_t, const float* __restrict__ sin_t,
                                               int rot, int interleaved, int pos, int d, int lane, T* dst) {
  HeadRegs<T, PARTS> r;
  r.load(x, w, cos_t, sin_t, rot, interleaved, pos, d, lane);
  r.finish(w != nullptr, eps, rot, interleaved, d, lane, dst);
}

}  // namespace xi
