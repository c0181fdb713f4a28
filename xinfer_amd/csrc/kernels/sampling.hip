// Sampling on the GPU: argmax, temperature, top-k, top-p, top-k-then-top-p, and the
// frequency/presence penalties, one workgroup per row of float32 logits.
//
// Reference: LogitsProcessor (/root/reference/src/utils/logits_processor.rs): strategies
// :12-18,48-65; p = softmax(logits / T) in float32 and a weighted draw :72-77,305-320;
// top-k keeps the k most probable :113-141; top-p keeps, in descending order, every
// token whose preceding cumulative mass is below p :82-111; top-k then top-p applies the
// cutoff to the renormalised top-k set :143-200; penalties :358-378.
//
// The kept set is described by a value v and a count: every probability above v, and the
// first `ties` tokens equal to v in index order (ties are common when logits come from
// bfloat16).  v is found without sorting, by a search over float bit patterns.  The draw
// takes a uniform number from the caller and walks the kept tokens in index order.
#include "common.h"

namespace xi {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / kWave;

__device__ __forceinline__ float block_sum_f(float v, float* s) { return block_sum<kSampleWaves>(v, s); }

__device__ __forceinline__ int block_sum_i(int v, int* s) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) s[threadIdx.x / kWave] = v;
  __syncthreads();
  int t = 0;
#pragma unroll
  for (int i = 0; i < kSampleWaves; ++i) t += s[i];
  return t;
}

__device__ __forceinline__ float block_max_f(float v, float* s) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) s[threadIdx.x / kWave] = v;
  __syncthreads();
  float t = s[0];
#pragma unroll
  for (int i = 1; i < kSampleWaves; ++i) t = fmaxf(t, s[i]);
  return t;
}

__device__ __forceinline__ float block_min_f(float v, float* s) { return -block_max_f(-v, s); }

// argmax with the lowest index winning ties
__device__ int block_argmax(const float* row, int V, float* sf, int* si) {
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = threadIdx.x; i < V; i += kSampleThreads) {
    const float v = row[i];
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
  }
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) {
    const float ob = __shfl_xor(best, off, kWave);
    const int oi = __shfl_xor(idx, off, kWave);
    if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
  }
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) { sf[threadIdx.x / kWave] = best; si[threadIdx.x / kWave] = idx; }
  __syncthreads();
  best = sf[0];
  idx = si[0];
  for (int i = 1; i < kSampleWaves; ++i)
    if (sf[i] > best || (sf[i] == best && si[i] < idx)) { best = sf[i]; idx = si[i]; }
  return idx;
}

__global__ __launch_bounds__(kSampleThreads) void argmax_kernel(const float* __restrict__ logits, int V,
                                                                int* __restrict__ out) {
  __shared__ float sf[kSampleWaves];
  __shared__ int si[kSampleWaves];
  const int r = block_argmax(logits + (size_t)blockIdx.x * V, V, sf, si);
  if (threadIdx.x == 0) out[blockIdx.x] = r;
}

// logits[row, t] -= count(t) * freq + presence for each token t among `recent[row, :]`
// (entries < 0 are padding).
__global__ void penalty_kernel(float* __restrict__ logits, int V, const int* __restrict__ recent, int n_recent,
                               const float* __restrict__ freq, const float* __restrict__ presence) {
  const int row = blockIdx.x;
  const float f = freq[row], p = presence[row];
  if (f == 0.f && p == 0.f) return;
  const int* rec = recent + (size_t)row * n_recent;
  for (int j = threadIdx.x; j < n_recent; j += blockDim.x) {
    const int t = rec[j];
    if (t < 0 || t >= V) continue;
    int count = 0;
    bool first = true;
    for (int i = 0; i < n_recent; ++i) {
      if (rec[i] == t) {
        ++count;
        if (i < j) first = false;
      }
    }
    if (first) logits[(size_t)row * V + t] -= (float)count * f + p;
  }
}

// count of p >= x and sum of p > x over the row
__device__ __forceinline__ int count_ge(const float* p, int V, float x, int* si) {
  int c = 0;
  for (int i = threadIdx.x; i < V; i += kSampleThreads) c += p[i] >= x;
  return block_sum_i(c, si);
}
__device__ __forceinline__ float sum_gt(const float* p, int V, float x, float* sf) {
  float s = 0.f;
  for (int i = threadIdx.x; i < V; i += kSampleThreads) s += p[i] > x ? p[i] : 0.f;
  return block_sum_f(s, sf);
}

__global__ __launch_bounds__(kSampleThreads) void sample_kernel(
    const float* __restrict__ logits, int V, const float* __restrict__ temperature,
    const int* __restrict__ top_k, const float* __restrict__ top_p, const float* __restrict__ uniform,
    float* __restrict__ probs, int* __restrict__ out) {
  __shared__ float sf[kSampleWaves];
  __shared__ int si[kSampleWaves];
  __shared__ float scan_f[kSampleThreads];
  __shared__ int scan_i[kSampleThreads];
  __shared__ int result;
  const int row = blockIdx.x;
  const float* lg = logits + (size_t)row * V;
  float* p = probs + (size_t)row * V;
  const float T = temperature[row];
  if (!(T >= 1e-7f)) {  // greedy (logits_processor.rs:53-58)
    const int r = block_argmax(lg, V, sf, si);
    if (threadIdx.x == 0) out[row] = r;
    return;
  }
  // unnormalised probabilities exp((l - max) / T); their sum is the total mass
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < V; i += kSampleThreads) mx = fmaxf(mx, lg[i]);
  mx = block_max_f(mx, sf);
  const float invT = 1.f / T;
  float z = 0.f;
  for (int i = threadIdx.x; i < V; i += kSampleThreads) {
    const float e = expf((lg[i] - mx) * invT);
    p[i] = e;
    z += e;
  }
  float mass = block_sum_f(z, sf);  // also orders the writes to p before the reads below

  // kept set: p > v, and the first `ties` tokens with p == v in index order
  float v = -1.f;
  int ties = 0;
  const int k = top_k[row];
  if (k > 0 && k < V) {
    // largest x with count(p >= x) >= k, i.e. the k-th largest value
    unsigned bits = 0;
    for (int b = 30; b >= 0; --b) {
      const unsigned cand = bits | (1u << b);
      if (count_ge(p, V, __uint_as_float(cand), si) >= k) bits = cand;
    }
    v = __uint_as_float(bits);
    const int n_gt = count_ge(p, V, __uint_as_float(bits + 1), si);
    ties = k - n_gt;
    mass = sum_gt(p, V, v, sf) + (float)ties * v;
  }
  const float tp = top_p[row];
  if (tp > 0.f && tp < 1.f) {
    const float target = tp * mass;
    // largest x with sum(p > x) >= target; the kept values are those above it
    unsigned bits = 0;
    if (sum_gt(p, V, 0.f, sf) >= target) {
      for (int b = 30; b >= 0; --b) {
        const unsigned cand = bits | (1u << b);
        if (sum_gt(p, V, __uint_as_float(cand), sf) >= target) bits = cand;
      }
      bits += 1;  // smallest x whose strictly-greater mass is below the target
    }
    const float x = fmaxf(__uint_as_float(bits), v);
    // the smallest kept value is the smallest actual value >= x
    float vm = INFINITY;
    for (int i = threadIdx.x; i < V; i += kSampleThreads)
      if (p[i] >= x && p[i] > 0.f) vm = fminf(vm, p[i]);
    vm = block_min_f(vm, sf);
    const float s_above = sum_gt(p, V, vm, sf);
    int cnt = count_ge(p, V, vm, si) - count_ge(p, V, __uint_as_float(__float_as_uint(vm) + 1), si);
    if (vm == v) cnt = ties;  // top-k already limited the ties at this value
    int keep = (int)ceilf((target - s_above) / vm);
    keep = max(1, min(keep, cnt));
    v = vm;
    ties = keep;
    mass = s_above + (float)ties * v;
  }

  // draw: walk the kept tokens in index order until the cumulative mass passes u * mass
  const float goal = uniform[row] * mass;
  const int per = (V + kSampleThreads - 1) / kSampleThreads;
  const int lo = min(V, (int)threadIdx.x * per), hi = min(V, lo + per);
  int my_ties = 0;
  for (int i = lo; i < hi; ++i) my_ties += (p[i] == v);
  scan_i[threadIdx.x] = my_ties;
  __syncthreads();
  if (threadIdx.x == 0) {  // exclusive prefix of tie counts (1024 adds; keeps the order exact)
    int run = 0;
    for (int t = 0; t < kSampleThreads; ++t) { const int c = scan_i[t]; scan_i[t] = run; run += c; }
    result = -1;
  }
  __syncthreads();
  int tie_rank = scan_i[threadIdx.x];
  float my_mass = 0.f;
  for (int i = lo; i < hi; ++i) {
    const float pi = p[i];
    if (pi > v) my_mass += pi;
    else if (pi == v) { if (tie_rank < ties) my_mass += pi; ++tie_rank; }
  }
  scan_f[threadIdx.x] = my_mass;
  __syncthreads();
  if (threadIdx.x == 0) {
    float run = 0.f;
    for (int t = 0; t < kSampleThreads; ++t) { const float c = scan_f[t]; scan_f[t] = run; run += c; }
  }
  __syncthreads();
  const float before = scan_f[threadIdx.x];
  if (my_mass > 0.f && before <= goal && goal < before + my_mass) {
    float run = before;
    tie_rank = scan_i[threadIdx.x];
    int pick = -1, last_kept = -1;
    for (int i = lo; i < hi; ++i) {
      const float pi = p[i];
      bool kept = pi > v;
      if (pi == v) { kept = tie_rank < ties; ++tie_rank; }
      if (!kept) continue;
      last_kept = i;
      run += pi;
      if (goal < run) { pick = i; break; }
    }
    result = pick >= 0 ? pick : last_kept;
  }
  __syncthreads();
  if (result < 0) {  // rounding left the goal at or beyond the total: take the last kept token
    int last = -1;
    tie_rank = scan_i[threadIdx.x];
    for (int i = lo; i < hi; ++i) {
      const float pi = p[i];
      bool kept = pi > v;
      if (pi == v) { kept = tie_rank < ties; ++tie_rank; }
      if (kept) last = i;
    }
    int best = last;
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) best = max(best, __shfl_xor(best, off, kWave));
    if ((threadIdx.x & (kWave - 1)) == 0) si[threadIdx.x / kWave] = best;
    __syncthreads();
    if (threadIdx.x == 0) {
      int b = -1;
      for (int i = 0; i < kSampleWaves; ++i) b = max(b, si[i]);
      result = b;
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) out[row] = result;
}

}  // namespace xi

using namespace xi;

extern "C" {

int xi_argmax(const float* logits, int rows, int V, int* out, hipStream_t stream) {
  XI_CHECK(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  argmax_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, V, out);
  XI_LAUNCH_CHECK("argmax");
  return 0;
}

int xi_apply_penalties(float* logits, int rows, int V, const int* recent, int n_recent, const float* freq,
                       const float* presence, hipStream_t stream) {
  XI_CHECK(rows >= 0 && V > 0 && n_recent >= 0, "penalties: bad sizes");
  if (rows == 0 || n_recent == 0) return 0;
  penalty_kernel<<<rows, 128, 0, stream>>>(logits, V, recent, n_recent, freq, presence);
  XI_LAUNCH_CHECK("penalties");
  return 0;
}

// probs: float32 scratch [rows, V].  uniform: one number in [0, 1) per row.
int xi_sample(const float* logits, int rows, int V, const float* temperature, const int* top_k,
              const float* top_p, const float* uniform, float* probs, int* out, hipStream_t stream) {
  XI_CHECK(rows >= 0 && V > 0, "sample: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  sample_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, V, temperature, top_k, top_p, uniform, probs, out);
  XI_LAUNCH_CHECK("sample");
  return 0;
}

}  // extern "C"
