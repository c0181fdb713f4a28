// Paged causal GQA attention, one workgroup per (token, query head), float32 math.
// It serves every case (prompt portions, decode tokens, windows, any head size) and is
// the attention of the 32-bit path; the bfloat16 path uses it where no faster kernel
// applies.  Keys of a token at position p are the cached positions lo..p of its own
// request, lo = max(0, p - window + 1), read through the request's block table.  K is
// [page, kv_head, offset, d]; V is the same or, with v_grouped, [page, kv_head, offset / 8, d, 8].
//
// Reference: PagedAttention::forward at /root/reference/src/models/layers/attention.rs:947-958
// (external kernel); golden formula tests/probes/compare_flashinfer_probe.py:51-73:
//   s[p'] = (q . k[p']) * scale for p' <= p, softmax over them in float32, o = sum a[p'] v[p'];
//   query head h reads kv head h / (nq / nkv).
//
// The order of every reduction is fixed by (position, window) alone: keys are taken in
// chunks of 64 starting at lo, chunk c goes to wave c % 4, and the four partial results
// are merged in wave order.
#include "common.h"

namespace xi {

constexpr int kMaxHeadDim = 256;
constexpr int kAttnWaves = 4;

template <typename T>
__global__ __launch_bounds__(kAttnWaves* kWave) void attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
    const int* __restrict__ block_tables, int max_pages, const int* __restrict__ tok_seq,
    const int* __restrict__ positions, T* __restrict__ out, float scale, int window, int page_size,
    int nq, int nkv, int d, int v_grouped) {
  __shared__ float q_s[kMaxHeadDim];
  __shared__ float acc_s[kAttnWaves][kMaxHeadDim];
  __shared__ float m_s[kAttnWaves], l_s[kAttnWaves];

  const int t = blockIdx.x;
  const int h = blockIdx.y;
  const int kvh = h / (nq / nkv);
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x / kWave;
  const int seq = tok_seq[t];
  const int pos = positions[t];
  const int lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  const int* bt = block_tables + (size_t)seq * max_pages;

  const T* qp = q + ((size_t)t * nq + h) * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) q_s[i] = to_float(qp[i]) * scale;
  __syncthreads();

  constexpr int NE = kMaxHeadDim / kWave;  // output dims per lane
  float acc[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) acc[e] = 0.f;
  float m = -INFINITY, l = 0.f;

  const int n_keys = pos - lo + 1;
  const int n_chunks = (n_keys + kWave - 1) / kWave;
  for (int c = wave; c < n_chunks; c += kAttnWaves) {
    const int key = lo + c * kWave + lane;
    const bool valid = key <= pos;
    int row = 0;  // row of this lane's key in the cache, in units of d elements
    int vrow = 0, voff = 0;  // grouped V: first row of the (page, kv head) block and the offset
    float s = -INFINITY;
    if (valid) {
      const int page = bt[key / page_size];
      row = (page * nkv + kvh) * page_size + key % page_size;
      vrow = (page * nkv + kvh) * d;
      voff = key % page_size;
      const T* kp = k_cache + (size_t)row * d;
      float dot = 0.f;
      for (int i = 0; i < d; ++i) dot = fmaf(q_s[i], to_float(kp[i]), dot);
      s = dot;
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - m_new) : 0.f;
    const float corr = expf(m - m_new);  // exp(-inf) = 0 on the first chunk
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int e = 0; e < NE; ++e) acc[e] *= corr;
    const int n_in_chunk = min(kWave, pos - (lo + c * kWave) + 1);
    for (int j = 0; j < n_in_chunk; ++j) {
      const float pj = __shfl(p, j, kWave);
      const int rj = __shfl(row, j, kWave);
      const int vrj = __shfl(vrow, j, kWave);
      const int voj = __shfl(voff, j, kWave);
      const T* vp = v_cache + (size_t)rj * d;
      const T* vtp = v_cache + (size_t)vrj * page_size + (size_t)(voj >> 3) * d * 8 + (voj & 7);  // [offset / 8, d, 8] block
#pragma unroll
      for (int e = 0; e < NE; ++e) {
        const int i = lane + e * kWave;
        if (i < d) {
          const float vv = v_grouped ? to_float(vtp[(size_t)i * 8]) : to_float(vp[i]);
          acc[e] = fmaf(pj, vv, acc[e]);
        }
      }
    }
  }
  if (lane == 0) {
    m_s[wave] = m;
    l_s[wave] = l;
  }
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int i = lane + e * kWave;
    if (i < d) acc_s[wave][i] = acc[e];
  }
  __syncthreads();
  float mm = m_s[0];
#pragma unroll
  for (int w = 1; w < kAttnWaves; ++w) mm = fmaxf(mm, m_s[w]);
  float f[kAttnWaves];
  float ll = 0.f;
#pragma unroll
  for (int w = 0; w < kAttnWaves; ++w) {
    f[w] = (m_s[w] == -INFINITY) ? 0.f : expf(m_s[w] - mm);
    ll += l_s[w] * f[w];
  }
  T* op = out + ((size_t)t * nq + h) * d;
  for (int i = threadIdx.x; i < d; i += blockDim.x) {
    float o = 0.f;
#pragma unroll
    for (int w = 0; w < kAttnWaves; ++w) o += acc_s[w][i] * f[w];
    op[i] = from_float<T>(o / ll);
  }
}

}  // namespace xi

using namespace xi;

extern "C" int xi_attention_generic(const void* q, const void* k_cache, const void* v_cache,
                                    int dtype, const int* block_tables, int max_pages,
                                    const int* tok_seq, const int* positions, void* out,
                                    float scale, int window, int page_size, int n_tok, int nq,
                                    int nkv, int d, int v_grouped, hipStream_t stream) {
  XI_CHECK(n_tok >= 0 && nq > 0 && nkv > 0 && page_size > 0 && max_pages > 0,
           "attention: bad sizes T=%d nq=%d nkv=%d page=%d max_pages=%d", n_tok, nq, nkv, page_size, max_pages);
  XI_CHECK(nq % nkv == 0, "attention: %d query heads are not a multiple of %d kv heads", nq, nkv);
  XI_CHECK(d > 0 && d <= kMaxHeadDim, "attention: head_dim %d is outside 1..%d", d, kMaxHeadDim);
  XI_CHECK(nq <= 65535, "attention: too many heads (%d)", nq);
  XI_CHECK(!v_grouped || page_size % 8 == 0, "attention: V in groups of eight keys needs pages of a multiple of 8 tokens, not %d", page_size);
  if (n_tok == 0) return 0;
  dim3 grid(n_tok, nq);
  if (dtype == kF32)
    attention_generic_kernel<float><<<grid, kAttnWaves * kWave, 0, stream>>>(
        (const float*)q, (const float*)k_cache, (const float*)v_cache, block_tables, max_pages,
        tok_seq, positions, (float*)out, scale, window, page_size, nq, nkv, d, v_grouped);
  else if (dtype == kBF16)
    attention_generic_kernel<bf16><<<grid, kAttnWaves * kWave, 0, stream>>>(
        (const bf16*)q, (const bf16*)k_cache, (const bf16*)v_cache, block_tables, max_pages,
        tok_seq, positions, (bf16*)out, scale, window, page_size, nq, nkv, d, v_grouped);
  else
    XI_CHECK(false, "attention: unknown dtype %d", dtype);
  XI_LAUNCH_CHECK("attention_generic");
  return 0;
}
