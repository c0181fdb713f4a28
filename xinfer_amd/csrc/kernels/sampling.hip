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
#include "no_alloc.h"

#include <atomic>
#include <mutex>

// Scratch of `xi_argmax_static`: per row and chunk the winner's value (float) and index (int).
// In host code this name is a stand-in, not a device address: host code uses the per-device
// pointer that hipGetSymbolAddress gives (`static_scratch` below), never the name itself.
constexpr int kStaticArgmaxRows = 256;
constexpr int kStaticArgmaxChunks = 32;
constexpr size_t kStaticArgmaxBytes = (size_t)kStaticArgmaxRows * kStaticArgmaxChunks * (sizeof(float) + sizeof(int));
static __device__ __align__(256) unsigned char scratch[kStaticArgmaxBytes];

namespace xi {

constexpr int kSampleThreads = 1024;
constexpr int kSampleWaves = kSampleThreads / kWave;

__device__ __forceinline__ float block_sum_f(float v, float* s) { return block_sum<kSampleWaves>(v, s); }

// The wave's largest value and, among equal ones, the lowest index, in every lane.
template <int OFF>
__device__ __forceinline__ void argmax_with(float& best, int& idx) {
  const float ob = lane_xor<OFF>(best);
  const int oi = lane_xor<OFF>(idx);
  if (ob > best || (ob == best && oi < idx)) { best = ob; idx = oi; }
}
__device__ __forceinline__ void wave_argmax(float& best, int& idx) {
  argmax_with<32>(best, idx);
  argmax_with<16>(best, idx);
  argmax_with<8>(best, idx);
  argmax_with<4>(best, idx);
  argmax_with<2>(best, idx);
  argmax_with<1>(best, idx);
}

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
  wave_argmax(best, idx);
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

// argmax in two stages, so that a few rows still use many compute units: stage one takes
// the row in `n_chunks` slices (lowest index wins ties within a slice), stage two merges the
// slices' winners in slice order (lowest index wins again).
__global__ __launch_bounds__(256) void argmax_partial_kernel(const float* __restrict__ logits, int V, int n_chunks,
                                                             float* __restrict__ pval, int* __restrict__ pidx) {
  __shared__ float sf[4];
  __shared__ int si[4];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int per = (V + n_chunks - 1) / n_chunks;
  const int lo = chunk * per, hi = min(V, lo + per);
  const float* r = logits + (size_t)row * V;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int i = lo + threadIdx.x; i < hi; i += 256) {
    const float v = r[i];
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
  }
  wave_argmax(best, idx);
  if ((threadIdx.x & (kWave - 1)) == 0) { sf[threadIdx.x / kWave] = best; si[threadIdx.x / kWave] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int i = 1; i < 4; ++i)
      if (sf[i] > best || (sf[i] == best && si[i] < idx)) { best = sf[i]; idx = si[i]; }
    pval[(size_t)row * n_chunks + chunk] = best;
    pidx[(size_t)row * n_chunks + chunk] = idx;
  }
}

__global__ __launch_bounds__(64) void argmax_merge_kernel(const float* __restrict__ pval, const int* __restrict__ pidx,
                                                          int n_chunks, int* __restrict__ out) {
  const int row = blockIdx.x;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  for (int c = threadIdx.x; c < n_chunks; c += kWave) {
    const float v = pval[(size_t)row * n_chunks + c];
    const int i = pidx[(size_t)row * n_chunks + c];
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
  }
  wave_argmax(best, idx);
  if (threadIdx.x == 0) out[row] = idx;
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

// ---- selection without sorting -------------------------------------------------------------
// Both cut-offs are "walk the values in descending order until a running total reaches a
// target": for top-k the total counts tokens, for top-p it adds probabilities.  Probabilities
// are non-negative floats, so their bit patterns order like the values, and the walk is done
// on a histogram of bit fields: 11 bits, then 11, then 9, each level one pass over the row
// that looks only at values inside the bin the level above chose.  Totals are integers
// (probabilities in units of 2^-40), so they do not depend on the order of the atomic adds.
typedef unsigned long long u64;
constexpr int kBins = 2048;
constexpr float kFix = 1099511627776.f;  // 2^40

__device__ __forceinline__ u64 shfl_up_u64(u64 v, int delta) {
  const unsigned lo = __shfl_up((unsigned)v, delta, kWave), hi = __shfl_up((unsigned)(v >> 32), delta, kWave);
  return ((u64)hi << 32) | lo;
}

// Bins hold weights w[0..n_bins).  Walking bins from the highest down, finds the bin b with
// (total of bins above b) < target <= (total of bins above b) + w[b]; returns it in *bin and
// the total above it in *above.  *bin = -1 if the target exceeds the total of all bins.
// scan: kSampleWaves + 2 u64 of LDS.
__device__ void find_crossing(const u64* w, int n_bins, u64 target, u64* scan, int* bin, u64* above) {
  const int per = (n_bins + kSampleThreads - 1) / kSampleThreads;
  const int top = n_bins - 1 - (int)threadIdx.x * per;      // this thread's highest bin
  u64 local = 0;
  for (int i = 0; i < per; ++i)
    if (top - i >= 0) local += w[top - i];
  // exclusive prefix over threads, thread 0 first
  u64 incl = local;
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
#pragma unroll
  for (int d = 1; d < kWave; d <<= 1) {
    const u64 o = shfl_up_u64(incl, d);
    if (lane >= d) incl += o;
  }
  __syncthreads();
  if (lane == kWave - 1) scan[wave] = incl;
  if (threadIdx.x == 0) {
    *bin = -1;
    *above = 0;
  }
  __syncthreads();
  u64 before = incl - local;
  for (int i = 0; i < wave; ++i) before += scan[i];
  u64 run = before;
  for (int i = 0; i < per; ++i) {
    const int b = top - i;
    if (b < 0) break;
    const u64 wb = w[b];
    if (run < target && target <= run + wb) {
      *bin = b;
      *above = run;
    }
    run += wb;
  }
  __syncthreads();
}

// Descends the three levels.  weighted: totals add probabilities (top-p), else count tokens
// (top-k).  Returns the bit pattern of the value at which the walk reaches `target` and, in
// *above, the total of everything strictly greater than that value; *at = number of tokens
// equal to it.  Returns 0xffffffff if the target exceeds the total over positive values.
__device__ unsigned select_value(const float* p, int V, bool weighted, u64 target, u64* hist, int* cnt_hist,
                                 u64* scan, int* s_bin, u64* s_above, u64* above, int* at) {
  unsigned prefix = 0;    // bits chosen so far (the high ones)
  u64 total_above = 0;
  const int shifts[3] = {20, 9, 0};
  const int widths[3] = {11, 11, 9};
  for (int level = 0; level < 3; ++level) {
    const int shift = shifts[level], n_bins = 1 << widths[level];
    for (int i = threadIdx.x; i < n_bins; i += kSampleThreads) {
      hist[i] = 0;
      cnt_hist[i] = 0;
    }
    __syncthreads();
    const unsigned hi_mask = level == 0 ? 0u : (0xffffffffu << (shift + widths[level]));
    for (int i = threadIdx.x; i < V; i += kSampleThreads) {
      const float pi = p[i];
      const unsigned bits = __float_as_uint(pi);
      if (bits == 0 || (bits & hi_mask) != (prefix & hi_mask)) continue;   // zero, or outside the chosen bin
      const int b = (bits >> shift) & (n_bins - 1);
      atomicAdd(&hist[b], weighted ? (u64)(pi * kFix) : (u64)1);
      if (level == 2) atomicAdd(&cnt_hist[b], 1);
    }
    __syncthreads();
    find_crossing(hist, n_bins, target - total_above, scan, s_bin, s_above);
    const int b = *s_bin;
    if (b < 0) return 0xffffffffu;
    prefix |= (unsigned)b << shift;
    total_above += *s_above;
    if (level == 2) *at = cnt_hist[b];
    __syncthreads();
  }
  *above = total_above;
  return prefix;
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
  __shared__ u64 hist[kBins];
  __shared__ int cnt_hist[kBins];
  __shared__ u64 scan64[kSampleWaves];
  __shared__ int s_bin;
  __shared__ u64 s_above;
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
    // the k-th largest value, the number of tokens above it, and how many of its ties fit
    u64 above;
    int at;
    const unsigned bits = select_value(p, V, false, (u64)k, hist, cnt_hist, scan64, &s_bin, &s_above, &above, &at);
    if (bits != 0xffffffffu) {   // else fewer than k tokens have a positive probability: keep them all
      v = __uint_as_float(bits);
      ties = k - (int)above;
      mass = sum_gt(p, V, v, sf) + (float)ties * v;
    }
  }
  const float tp = top_p[row];
  if (tp > 0.f && tp < 1.f) {
    const float target = tp * mass;
    // the smallest value whose strictly greater mass is still below the target: the last
    // token kept in descending order has it (logits_processor.rs:82-111)
    u64 above;
    int at = 0;
    const unsigned bits = select_value(p, V, true, (u64)(target * kFix), hist, cnt_hist, scan64, &s_bin, &s_above,
                                       &above, &at);
    if (bits != 0xffffffffu) {
      float vm = __uint_as_float(bits);
      int cnt = at;
      if (vm <= v) {   // top-k already cut higher (or here): its bound and its ties stand
        vm = v;
        cnt = ties;
      }
      const float s_above_f = sum_gt(p, V, vm, sf);
      int keep = (int)ceilf((target - s_above_f) / vm);
      keep = max(1, min(keep, cnt));
      v = vm;
      ties = keep;
      mass = s_above_f + (float)ties * v;
    }
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

// Chunks stage one of the argmax cuts a row of V logits into.
int xi_argmax_chunks(int V) { return V >= 16384 ? 32 : 1; }

// pval / pidx: scratch [rows, xi_argmax_chunks(V)] (unused when that is 1).
int xi_argmax(const float* logits, int rows, int V, int* out, float* pval, int* pidx, hipStream_t stream) {
  XI_CHECK(rows >= 0 && V > 0, "argmax: bad sizes rows=%d V=%d", rows, V);
  if (rows == 0) return 0;
  const int n_chunks = xi_argmax_chunks(V);
  if (n_chunks == 1) {
    argmax_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, V, out);
    XI_LAUNCH_CHECK("argmax");
    return 0;
  }
  XI_CHECK(pval != nullptr && pidx != nullptr && rows <= 65535, "argmax: scratch for %d chunks is missing", n_chunks);
  argmax_partial_kernel<<<dim3(n_chunks, rows), 256, 0, stream>>>(logits, V, n_chunks, pval, pidx);
  XI_LAUNCH_CHECK("argmax_partial");
  argmax_merge_kernel<<<rows, 64, 0, stream>>>(pval, pidx, n_chunks, out);
  XI_LAUNCH_CHECK("argmax_merge");
  return 0;
}

// ---- the entry point that allocates nothing (no_alloc.h) ----------------------------------
// Each GPU holds its own copy of `scratch` at its own address; the address is asked for once
// per device, with that device current, and kept.
constexpr int kStaticMaxDevices = 64;
static std::atomic<void*> g_static_scratch[kStaticMaxDevices];
static std::mutex g_static_mutex;

// The array's address on the current device.  The first call on a device asks the runtime for it
// (under the mutex, once); later calls read what was kept and make no runtime call but hipGetDevice.
static int static_scratch(unsigned char** ptr) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  XI_CHECK(e == hipSuccess, "argmax_static: hipGetDevice failed: %s", hipGetErrorString(e));
  XI_CHECK(dev >= 0 && dev < kStaticMaxDevices, "argmax_static: device %d is beyond the %d this library keeps", dev,
           kStaticMaxDevices);
  void* p = g_static_scratch[dev].load(std::memory_order_acquire);
  if (p == nullptr) {
    std::lock_guard<std::mutex> lock(g_static_mutex);
    p = g_static_scratch[dev].load(std::memory_order_relaxed);
    if (p == nullptr) {
      e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      XI_CHECK(e == hipSuccess && p != nullptr, "argmax_static: hipGetSymbolAddress failed on device %d: %s", dev,
               hipGetErrorString(e));
      g_static_scratch[dev].store(p, std::memory_order_release);
    }
  }
  *ptr = static_cast<unsigned char*>(p);
  return 0;
}

int xi_argmax_static_init() {
  unsigned char* base = nullptr;
  return static_scratch(&base);
}

int xi_argmax_static_max_rows() { return kStaticArgmaxRows; }

int xi_argmax_static(const float* logits, int rows, int V, int* out, hipStream_t stream) {
  XI_CHECK(rows >= 0 && V > 0, "argmax_static: bad sizes rows=%d V=%d", rows, V);
  XI_CHECK(rows <= kStaticArgmaxRows, "argmax_static: %d rows are more than the %d the fixed scratch holds", rows,
           kStaticArgmaxRows);
  if (rows == 0) return 0;
  XI_CHECK(logits != nullptr && out != nullptr, "argmax_static: logits or out is null");
  const int n_chunks = xi_argmax_chunks(V);
  XI_CHECK(n_chunks <= kStaticArgmaxChunks, "argmax_static: %d chunks are more than the %d the fixed scratch holds",
           n_chunks, kStaticArgmaxChunks);
  if (n_chunks == 1) {
    argmax_kernel<<<rows, kSampleThreads, 0, stream>>>(logits, V, out);
    XI_LAUNCH_CHECK("argmax_static");
    return 0;
  }
  unsigned char* base = nullptr;
  if (int rc = static_scratch(&base)) return rc;
  float* pval = reinterpret_cast<float*>(base);
  int* pidx = reinterpret_cast<int*>(base + (size_t)kStaticArgmaxRows * kStaticArgmaxChunks * sizeof(float));
  // stage one writes all rows * n_chunks slots that stage two reads: the last call's contents never show
  argmax_partial_kernel<<<dim3(n_chunks, rows), 256, 0, stream>>>(logits, V, n_chunks, pval, pidx);
  XI_LAUNCH_CHECK("argmax_static_partial");
  argmax_merge_kernel<<<rows, 64, 0, stream>>>(pval, pidx, n_chunks, out);
  XI_LAUNCH_CHECK("argmax_static_merge");
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
