// Sampling with a small top-k (the reference's default is top-k 32, then top-p 0.95, at
// temperature 0.7: /root/reference/src/core/runner.rs:1803-1854) without a pass of one
// workgroup over the whole vocabulary: the k most probable tokens are found in two stages that
// use the whole chip, and everything after that (softmax over the k, the top-p cut, the draw)
// is about k <= 64 numbers.  Same rules as sampling.hip: larger logit first, lower token id
// first among equal logits; top-p keeps, in that order, every token whose preceding cumulative
// mass is below p times the mass of the top-k set (logits_processor.rs:82-111, 143-200); the
// draw walks the kept tokens in token order with the caller's uniform number.  A row with a
// temperature below 1e-7 takes its most probable token (logits_processor.rs:53-58).
//
// Stage one: a workgroup takes 2560 logits of a row (10 a thread, in registers) and hands on its
// k first, found one a round (a round: every thread's best, the workgroup's best of those, its
// owner drops it).  Stage two: one workgroup a row takes the k first of all candidates the same
// way and finishes the row.
#include "common.h"

namespace xi {

constexpr int kTkThreads = 256;
constexpr int kTkWaves = kTkThreads / kWave;
constexpr int kTkMaxK = 64;
constexpr int kTkPer = 10;                        // logits a thread of stage one holds
constexpr int kTkChunk = kTkThreads * kTkPer;     // logits a workgroup of stage one takes
constexpr int kTkCand = 16;                       // candidates a thread of stage two holds
constexpr int kTkMaxChunks = kTkThreads * kTkCand / kTkMaxK;   // 64: vocabularies up to 163,840
constexpr int kTkNone = 0x7fffffff;               // index of "no element"

__device__ __forceinline__ bool tk_before(float a, int ia, float b, int ib) { return a > b || (a == b && ia < ib); }

// The workgroup's k first (value, index) pairs in the order of tk_before, into out_v / out_i
// (LDS, [kTkMaxK]); a thread holds E pairs, absent ones as (-inf, kTkNone).  s_v / s_i: LDS
// [2][kTkWaves].  One barrier a round; the caller synchronizes before it reads the result.
template <int E>
__device__ void tk_extract(float (&v)[E], int (&ix)[E], int k, float* out_v, int* out_i, float* s_v, int* s_i) {
  const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
  for (int it = 0; it < k; ++it) {
    float bv = -INFINITY;
    int bi = kTkNone;
#pragma unroll
    for (int e = 0; e < E; ++e)
      if (tk_before(v[e], ix[e], bv, bi)) { bv = v[e]; bi = ix[e]; }
#pragma unroll
    for (int off = kWave / 2; off > 0; off >>= 1) {
      const float ov = __shfl_xor(bv, off, kWave);
      const int oi = __shfl_xor(bi, off, kWave);
      if (tk_before(ov, oi, bv, bi)) { bv = ov; bi = oi; }
    }
    const int par = (it & 1) * kTkWaves;
    if (lane == 0) { s_v[par + wave] = bv; s_i[par + wave] = bi; }
    __syncthreads();
    float wv = s_v[par];
    int wi = s_i[par];
#pragma unroll
    for (int w = 1; w < kTkWaves; ++w)
      if (tk_before(s_v[par + w], s_i[par + w], wv, wi)) { wv = s_v[par + w]; wi = s_i[par + w]; }
    if (threadIdx.x == 0) { out_v[it] = wv; out_i[it] = wi == kTkNone ? -1 : wi; }
    if (wi != kTkNone) {
#pragma unroll
      for (int e = 0; e < E; ++e)
        if (ix[e] == wi) { v[e] = -INFINITY; ix[e] = kTkNone; }
    }
  }
}

// params: float32 [4, R] = temperature, top_k, top_p, uniform number of every row
__device__ __forceinline__ int tk_k_of(const float* params, int R, int row) {
  if (!(params[row] >= 1e-7f)) return 1;     // a greedy row: its first token alone
  int k = (int)params[R + row];
  return k < 1 ? 1 : (k > kTkMaxK ? kTkMaxK : k);
}

__global__ __launch_bounds__(kTkThreads) void topk_chunk_kernel(const float* __restrict__ logits, int V, int n_chunks,
                                                                const float* __restrict__ params, int R,
                                                                float* __restrict__ cand_v, int* __restrict__ cand_i) {
  __shared__ float out_v[kTkMaxK];
  __shared__ int out_i[kTkMaxK];
  __shared__ float s_v[2 * kTkWaves];
  __shared__ int s_i[2 * kTkWaves];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const int k = tk_k_of(params, R, row);
  const float* lg = logits + (size_t)row * V;
  float v[kTkPer];
  int ix[kTkPer];
#pragma unroll
  for (int e = 0; e < kTkPer; ++e) {
    const int i = chunk * kTkChunk + e * kTkThreads + (int)threadIdx.x;
    const bool ok = i < V;
    v[e] = ok ? lg[i] : -INFINITY;
    ix[e] = ok ? i : kTkNone;
  }
  tk_extract<kTkPer>(v, ix, k, out_v, out_i, s_v, s_i);
  __syncthreads();
  if ((int)threadIdx.x < k) {
    const size_t at = ((size_t)row * n_chunks + chunk) * kTkMaxK + threadIdx.x;
    cand_v[at] = out_v[threadIdx.x];
    cand_i[at] = out_i[threadIdx.x];
  }
}

__global__ __launch_bounds__(kTkThreads) void topk_finish_kernel(const float* __restrict__ cand_v,
                                                                 const int* __restrict__ cand_i, int n_chunks,
                                                                 const float* __restrict__ params, int R,
                                                                 int* __restrict__ out) {
  __shared__ float top_v[kTkMaxK];
  __shared__ int top_i[kTkMaxK];
  __shared__ float ps[kTkMaxK];
  __shared__ int order[kTkMaxK];
  __shared__ float s_v[2 * kTkWaves];
  __shared__ int s_i[2 * kTkWaves];
  __shared__ int s_m;
  const int row = blockIdx.x;
  const int k = tk_k_of(params, R, row);
  const int n = n_chunks * k;                  // candidates: k of every chunk
  float v[kTkCand];
  int ix[kTkCand];
#pragma unroll
  for (int e = 0; e < kTkCand; ++e) {
    const int c = e * kTkThreads + (int)threadIdx.x;
    v[e] = -INFINITY;
    ix[e] = kTkNone;
    if (c < n) {
      const size_t at = ((size_t)row * n_chunks + c / k) * kTkMaxK + c % k;
      const int id = cand_i[at];
      if (id >= 0) { v[e] = cand_v[at]; ix[e] = id; }
    }
  }
  tk_extract<kTkCand>(v, ix, k, top_v, top_i, s_v, s_i);
  __syncthreads();
  const float T = params[row];
  if (!(T >= 1e-7f)) {
    if (threadIdx.x == 0) out[row] = top_i[0] < 0 ? 0 : top_i[0];
    return;
  }
  // unnormalised probabilities of the k, largest first: exp((l - max) / T)
  if ((int)threadIdx.x < kTkMaxK) {
    const int j = threadIdx.x;
    const bool there = j < k && top_i[j] >= 0 && top_v[j] > -INFINITY;
    ps[j] = there ? expf((top_v[j] - top_v[0]) / T) : 0.f;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float mass = 0.f;
    for (int j = 0; j < k; ++j) mass += ps[j];
    const float tp = params[2 * R + row];
    int m = 0;
    if (tp > 0.f && tp < 1.f) {
      float cum = 0.f;
      for (int j = 0; j < k; ++j) {
        if (cum >= tp * mass) break;
        cum += ps[j];
        ++m;
      }
    } else {
      m = k;
    }
    while (m > 1 && !(ps[m - 1] > 0.f)) --m;   // tokens that are not there carry no mass
    s_m = m < 1 ? 1 : m;
  }
  __syncthreads();
  const int m = s_m;
  // the kept tokens in token order: a token's place is the number of kept tokens with a lower id
  if ((int)threadIdx.x < m) {
    const int mine = top_i[threadIdx.x];
    int rank = 0;
    for (int i = 0; i < m; ++i) rank += top_i[i] < mine;
    order[rank] = threadIdx.x;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    float total = 0.f;
    for (int r = 0; r < m; ++r) total += ps[order[r]];
    const float goal = params[3 * R + row] * total;
    float run = 0.f;
    int pick = -1;
    for (int r = 0; r < m; ++r) {
      run += ps[order[r]];
      if (goal < run) { pick = order[r]; break; }
    }
    if (pick < 0) pick = order[m - 1];       // rounding left the goal at the total: the last kept token
    const int id = top_i[pick];
    out[row] = id < 0 ? 0 : id;
  }
}

}  // namespace xi

using namespace xi;

extern "C" {

// Chunks of stage one for a vocabulary of V logits; 0 if the vocabulary is too large for this path.
int xi_sample_topk_chunks(int V) {
  if (V < 1) return 0;
  const int c = (V + kTkChunk - 1) / kTkChunk;
  return c <= kTkMaxChunks ? c : 0;
}

int xi_sample_topk_max_k() { return kTkMaxK; }

// logits float32 [R, V]; params float32 [4, R] = temperature, top_k (1..64; ignored for greedy
// rows), top_p, uniform number; cand_v / cand_i: scratch [R, chunks, 64]; out int32 [R].
int xi_sample_topk(const float* logits, int R, int V, const float* params, float* cand_v, int* cand_i, int* out,
                   hipStream_t stream) {
  XI_CHECK(R >= 0 && V > 0, "sample_topk: bad sizes rows=%d V=%d", R, V);
  const int chunks = xi_sample_topk_chunks(V);
  XI_CHECK(chunks > 0, "sample_topk: a vocabulary of %d is too large (at most %d)", V, kTkMaxChunks * kTkChunk);
  XI_CHECK(R <= 65535, "sample_topk: %d rows are too many for one launch", R);
  if (R == 0) return 0;
  topk_chunk_kernel<<<dim3(chunks, R), kTkThreads, 0, stream>>>(logits, V, chunks, params, R, cand_v, cand_i);
  XI_LAUNCH_CHECK("sample_topk");
  topk_finish_kernel<<<R, kTkThreads, 0, stream>>>(cand_v, cand_i, chunks, params, R, out);
  XI_LAUNCH_CHECK("sample_topk");
  return 0;
}

}  // extern "C"
