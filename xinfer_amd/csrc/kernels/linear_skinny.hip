// y[M,N] = x[M,K] @ w[N,K]^T in bfloat16 for few rows (decode batches, M <= 64): bound by
// the one pass over w, so the kernel is a streaming read of w through the matrix cores.
//
// A workgroup owns R output features (rows of w; R <= 16*RT, any number, so that the grid can
// be a multiple of the compute units) and one of KS slices of K.  Its NW waves take
// consecutive parts of the slice and merge through LDS in a fixed order, so an output
// element's value depends on (K, KS, NW) alone, never on M, on RT, on R or on what else is in
// the batch.  A wave keeps U steps of loads in flight: a step's registers are loaded again, U
// steps ahead, right after its products.  Per 32-wide k step a wave issues v_mfma_f32_16x16x32_bf16 with A = 16 rows
// of w (lane l: row l%16, k group l/16, one 16-byte load) and B = x^T (lane l: token l%16,
// same k group), for RT row tiles and MT tiles of 16 tokens: every x operand is used RT
// times and every w operand MT times.  x is small and is read from L2.
//
// With KS > 1 the workgroups of different slices write float32 partial sums [KS, M, N]; the
// consumer (the fused add + RMSNorm) adds them in slice order.  That gives narrow outputs
// (N = hidden size) enough workgroups for every compute unit and still lets a workgroup
// keep several row tiles per x operand.
//
// GATED: w is [2N, K] = [gate; up]; the workgroup computes rows n (gate) and N + n (up)
// and stores silu(gate) * up, float32 math and one rounding, so the packed [M, 2N]
// intermediate of the feed-forward never goes to memory.
//
// Reference call sites: candle matmul in /root/reference/src/models/layers/linear.rs:76-124
// (vendor BLAS); fused gate/up + silu_and_mul in /root/reference/src/models/layers/mlp.rs:613-633.
#include "common.h"
#include <cmath>
#include <type_traits>

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

__device__ __forceinline__ bf16x8 ldg8(const bf16* p) { return *reinterpret_cast<const bf16x8*>(p); }
__device__ __forceinline__ bf16x8 zeros8() {
  bf16x8 z;
#pragma unroll
  for (int i = 0; i < 8; ++i) z[i] = (__bf16)0.f;
  return z;
}

// A norm folded into the two products around it (few rows, MT = 1).  The product before the
// norm (MODE 1, kFoldOut) adds its result into the float32 residual stream, writes
// xg = round(stream * g) with the norm's weight g, and the sum of squares of its part of every
// row, one per workgroup.  The product after the norm (MODE 2, kFoldIn) takes xg as its x and
// multiplies each row of its result by rsqrt(sum of the parts / H + eps): the same value as
// norming first, up to where the one rounding to bfloat16 happens, and without the norm's own
// kernel between two kernels that stream weights.
struct SkinnyFold {
  float* resid;         // kFoldOut: [M, N] float32, updated in place
  const float* g;       // kFoldOut: [N] weight of the norm that follows
  bf16* xg;             // kFoldOut: [M, N]
  float* ss_out;        // kFoldOut: [M, gridDim.x]
  const float* ss_in;   // kFoldIn: [M, parts]
  int parts;            // kFoldIn
  float eps;            // kFoldIn
  float inv_h;          // kFoldIn: 1 / length of the normed rows
};
constexpr int kFoldNone = 0, kFoldOut = 1, kFoldIn = 2;

template <int MT, int RT, int NW, int U, bool GATED, typename TO, int MODE>
__global__ __launch_bounds__(NW * 64) void linear_skinny_kernel(const bf16* __restrict__ x,
                                                                const bf16* __restrict__ w,
                                                                TO* __restrict__ y, int M, int N, int K,
                                                                int steps_per_slice, int R, SkinnyFold fold) {
  static_assert(!GATED || RT % 2 == 0, "the gated form pairs gate tiles with up tiles");
  static_assert(MODE == kFoldNone || (MT == 1 && NW == 8), "a folded norm: up to 16 rows, 8 waves");
  static_assert(MODE != kFoldOut || !GATED, "the product before a norm is a plain one");
  // The waves' sums are merged through LDS a chunk of PC output tiles (gated: pairs of a gate
  // and an up tile) at a time, so that the buffer stays within 64 KB whatever RT and MT are.
  constexpr int H = NW / 2;                      // waves whose sums are left after the first round
  constexpr int TP = GATED ? 2 : 1;              // tiles of w per output tile
  constexpr int PAIRS = RT / TP;
  static_assert(H * TP * MT <= 64, "one output tile's sums must fit in 64 KB of LDS");
  constexpr int PC = (64 / (H * TP * MT)) < PAIRS ? (64 / (H * TP * MT)) : PAIRS;
  __shared__ float red[H * PC * TP * MT * 256];
  static_assert(MODE != kFoldOut || PC == PAIRS, "the product before a norm stores in one pass");
  __shared__ float fold_lds[MODE == kFoldOut ? 16 * 16 * RT : 16];   // squares [token][n], or 1/rms [token]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  // kFoldIn: 32 threads per row add up the parts of its sum of squares; the loads start now, the
  // sum is taken after the products
  constexpr int kSsLoads = 16;   // 32 threads x 16 loads: up to 512 parts of a row's sum
  float ss_mine[kSsLoads];
  if constexpr (MODE == kFoldIn) {
    const int token = threadIdx.x >> 5, sub = threadIdx.x & 31;
#pragma unroll
    for (int i = 0; i < kSsLoads; ++i) {
      const int p = sub + 32 * i;
      ss_mine[i] = (token < M && p < fold.parts) ? fold.ss_in[(size_t)token * fold.parts + p] : 0.f;
    }
  }
  // The workgroup owns output features n0 .. n0 + R - 1 (R <= 16 * PAIRS, any number: the grid
  // can then be a multiple of the compute units whatever N is).  Lanes past its last feature
  // read that feature's row again (the same address in one instruction costs nothing) and their
  // results are dropped.
  const int n0 = blockIdx.x * R;
  const int ks = blockIdx.y;
  const int n_last = min(n0 + R, N) - 1;

  const bf16* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    const int tl = GATED ? (t < RT / 2 ? t : t - RT / 2) : t;     // tile among the workgroup's features
    int n = n0 + 16 * tl + r;
    if (n > n_last) n = n_last;
    const int row = (GATED && t >= RT / 2) ? N + n : n;
    wp[t] = w + (size_t)row * K + 8 * j;
  }
  const bf16* xp[MT];
#pragma unroll
  for (int m = 0; m < MT; ++m) {
    int tok = 16 * m + r;
    if (tok > M - 1) tok = M - 1;
    xp[m] = x + (size_t)tok * K + 8 * j;
  }

  f32x4 acc[RT][MT];
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[t][m] = f32x4{0.f, 0.f, 0.f, 0.f};

  const int steps = (K + 31) / 32;      // k steps of 32
  const int steps_full = K / 32;        // steps in which every lane's 8 elements exist
  const int slice0 = ks * steps_per_slice;
  const int slice1 = min(steps, slice0 + steps_per_slice);
  const int per = (steps_per_slice + NW - 1) / NW;
  const int s0 = slice0 + wave * per;
  const int s1 = min(slice1, s0 + per);
  const int s_fast = min(s1, steps_full);
  int s = s0;
  // UU steps at once: all their loads are issued before the first product
  auto block = [&](auto uu_tag) {
    constexpr int UU = decltype(uu_tag)::value;
    bf16x8 a[RT][UU], b[MT][UU];
#pragma unroll
    for (int u = 0; u < UU; ++u) {
#pragma unroll
      for (int t = 0; t < RT; ++t) a[t][u] = ldg8(wp[t] + 32 * (s + u));
#pragma unroll
      for (int m = 0; m < MT; ++m) b[m][u] = ldg8(xp[m] + 32 * (s + u));
    }
#pragma unroll
    for (int u = 0; u < UU; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], b[m][u], acc[t][m], 0, 0, 0);
    s += UU;
  };
  // The main part keeps U steps of loads in flight all the time: a step's registers are loaded
  // again, U steps ahead, right after its products.  The sums run in the same order as in
  // `block`, so the result does not depend on which of the two forms ran.
  if (s + 2 * U <= s_fast) {
    bf16x8 a[RT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < RT; ++t) a[t][u] = ldg8(wp[t] + 32 * (s + u));
#pragma unroll
      for (int m = 0; m < MT; ++m) b[m][u] = ldg8(xp[m] + 32 * (s + u));
    }
    for (; s + 2 * U <= s_fast; s += U) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int m = 0; m < MT; ++m)
            acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], b[m][u], acc[t][m], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < RT; ++t) a[t][u] = ldg8(wp[t] + 32 * (s + U + u));
#pragma unroll
        for (int m = 0; m < MT; ++m) b[m][u] = ldg8(xp[m] + 32 * (s + U + u));
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], b[m][u], acc[t][m], 0, 0, 0);
    s += U;
  }
  while (s + U <= s_fast) block(std::integral_constant<int, U>{});
  if constexpr (U >= 8) {
    if (s + 4 <= s_fast) block(std::integral_constant<int, 4>{});
  }
  if constexpr (U >= 4) {
    if (s + 2 <= s_fast) block(std::integral_constant<int, 2>{});
  }
  for (; s < s1; ++s) {  // the rest, one step at a time; K % 8 == 0 so a lane's chunk exists or not
    const bool ok = 32 * s + 8 * j < K;
#pragma unroll
    for (int t = 0; t < RT; ++t) {
      const bf16x8 a = ok ? ldg8(wp[t] + 32 * s) : zeros8();
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        const bf16x8 b = ok ? ldg8(xp[m] + 32 * s) : zeros8();
        acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t][m], 0, 0, 0);
      }
    }
  }

  // merge the waves in a fixed order: wave w + NW/2 hands its sums to wave w, then all threads
  // add the NW/2 sums that are left, in wave order, and store.  A lane's 4 values of a tile:
  // token r, features 4j..4j+3.  Slot of (wave wv, output tile q of the chunk, part tp, token
  // tile m): ((wv * PC + q) * TP + tp) * MT + m.
  TO* yk = y + (size_t)ks * M * N;   // this slice's partial sums (ks is 0 without slices)
  if constexpr (MODE == kFoldIn) {   // read after the barriers of the merge below
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kSsLoads; ++i) t += ss_mine[i];
    t += lane_xor<16>(t);
    t += lane_xor<8>(t);
    t += lane_xor<4>(t);
    t += lane_xor<2>(t);
    t += lane_xor<1>(t);
    if ((threadIdx.x & 31) == 0) fold_lds[threadIdx.x >> 5] = rsqrtf(t * fold.inv_h + fold.eps);
  }
#pragma unroll
  for (int p0 = 0; p0 < PAIRS; p0 += PC) {
    if (p0 > 0) __syncthreads();     // the chunk before has been read
    if (wave >= H) {
#pragma unroll
      for (int q = 0; q < PC; ++q)
#pragma unroll
        for (int tp = 0; tp < TP; ++tp)
#pragma unroll
          for (int m = 0; m < MT; ++m)
            if (p0 + q < PAIRS)
              *reinterpret_cast<f32x4*>(&red[((((wave - H) * PC + q) * TP + tp) * MT + m) * 256 + lane * 4]) =
                  acc[tp * PAIRS + (p0 + q < PAIRS ? p0 + q : 0)][m];
    }
    __syncthreads();
    if (wave < H) {
#pragma unroll
      for (int q = 0; q < PC; ++q)
#pragma unroll
        for (int tp = 0; tp < TP; ++tp)
#pragma unroll
          for (int m = 0; m < MT; ++m)
            if (p0 + q < PAIRS) {
              f32x4* slot = reinterpret_cast<f32x4*>(&red[(((wave * PC + q) * TP + tp) * MT + m) * 256 + lane * 4]);
              const f32x4 o = *slot;
              f32x4 sum = acc[tp * PAIRS + (p0 + q < PAIRS ? p0 + q : 0)][m];
              sum[0] += o[0];
              sum[1] += o[1];
              sum[2] += o[2];
              sum[3] += o[3];
              *slot = sum;      // the same lane wrote and reads this slot: no barrier in between
            }
    }
    __syncthreads();
    const int pairs_here = PAIRS - p0 < PC ? PAIRS - p0 : PC;
    for (int idx = threadIdx.x; idx < pairs_here * MT * 256; idx += NW * 64) {
      const int tile = idx >> 8, e = idx & 255;
      const int q = tile / MT, m = tile - q * MT;
      const int ln = e >> 2, v = e & 3;
      const int token = 16 * m + (ln & 15), n = n0 + 16 * (p0 + q) + 4 * (ln >> 4) + v;
      float a0 = 0.f, a1 = 0.f;
#pragma unroll
      for (int wv = 0; wv < H; ++wv) {
        a0 += red[(((wv * PC + q) * TP) * MT + m) * 256 + e];
        if (GATED) a1 += red[(((wv * PC + q) * TP + 1) * MT + m) * 256 + e];
      }
      if constexpr (MODE == kFoldIn) {
        const float inv = fold_lds[token];
        a0 *= inv;
        a1 *= inv;
      }
      const bool mine = n <= n_last;      // a feature of this workgroup that exists
      if constexpr (MODE == kFoldOut) {
        float sq = 0.f;
        if (token < M && mine) {
          const float rr = fold.resid[(size_t)token * N + n] + a0;
          fold.resid[(size_t)token * N + n] = rr;
          fold.xg[(size_t)token * N + n] = from_float<bf16>(rr * fold.g[n]);
          sq = rr * rr;
        }
        fold_lds[token * (16 * RT) + (n - n0)] = sq;
      } else {
        if (token < M && mine)
          yk[(size_t)token * N + n] = from_float<TO>(GATED ? a0 / (1.f + __expf(-a0)) * a1 : a0);
      }
    }
  }
  if constexpr (MODE == kFoldOut) {   // a row's squares summed in the order of n
    __syncthreads();
    if (threadIdx.x < 16 && (int)threadIdx.x < M) {
      float t = 0.f;
      for (int i = 0; i < 16 * RT; ++i) t += fold_lds[threadIdx.x * (16 * RT) + i];
      fold.ss_out[(size_t)threadIdx.x * gridDim.x + blockIdx.x] = t;
    }
  }
}

struct SkinnyPlan {
  int ks;    // slices of K across workgroups
  int nw;    // waves per workgroup
  int rt;    // row tiles of w per workgroup (the kernel's shape)
  int rows;  // output features per workgroup, at most 16 * rt (gated: 8 * rt)
};

// Shapes that are built: 16 waves leave registers for 2 row tiles, 8 row tiles for 32 tokens.
static bool skinny_shape_ok(int rt, int nw, int mt, bool gated) {
  if (gated ? !(rt == 2 || rt == 4 || rt == 6 || rt == 8) : !(rt == 1 || rt == 2 || rt == 3 || rt == 4 || rt == 6 || rt == 8))
    return false;
  if (nw == 16 && rt > 2) return false;
  if (rt == 8 && mt > 2) return false;
  return true;
}

// ks and nw fix the order of the sums: they come from (N, K) and the caller's wish alone.
// rt and rows only say which workgroup computes what, and are chosen for speed.  Measured on
// MI355X: a workgroup reads its x operands from L2 once for all its rows of w, and such a read
// costs about 0.6 of a read of w from memory, so more rows of w pay with more rows of x; the
// stream of w itself slows by about 4% per further row tile; and a grid that is no multiple of
// the 256 compute units leaves some of them idle at the end, which is why a workgroup may own
// a number of features that is no multiple of 16 (N = 5120: 20 each make 256 workgroups).
static SkinnyPlan plan_skinny(int M, int N, int K, bool gated, bool allow_split) {
  SkinnyPlan p;
  const int tiles = (N + 15) / 16;       // output tiles (gated: each a gate tile and an up tile)
  p.ks = 1;
  if (allow_split && !gated) {
    p.ks = (1024 + tiles - 1) / tiles;
    if (p.ks > 4) p.ks = 4;
    while (p.ks > 1 && K / p.ks < 512) --p.ks;
  }
  p.nw = 8;
  const int mt = (M + 15) / 16;
  const int per = gated ? 2 : 1;         // tiles of w per output tile
  double best = 0.;
  p.rt = per;
  p.rows = 16;
  for (int q = 1; q <= 8; ++q) {         // output tiles per workgroup
    const int rt = q * per;
    if (rt > 8 || !skinny_shape_ok(rt, p.nw, mt, gated)) continue;
    const int cap = 16 * q;
    const int g_full = (N + cap - 1) / cap;
    // whole tiles, or the next grids that are multiples of 128 and of 256 workgroups
    const int grids[3] = {g_full, (g_full * p.ks + 127) / 128 * 128 / p.ks, (g_full * p.ks + 255) / 256 * 256 / p.ks};
    for (int c = 0; c < 3; ++c) {
      if (grids[c] < g_full) continue;
      const int rows = c == 0 ? cap : (N + grids[c] - 1) / grids[c];
      if (rows < 1 || rows > cap) continue;
      const double g = (double)((N + rows - 1) / rows) * p.ks / 256.;
      const double idle = g >= 1. ? ceil(g) / g : pow(g, -0.6);
      const double cost = idle * (1. + 0.04 * (rt - 1) + 0.6 * (double)M / (rows * per));
      if (best == 0. || cost < best * 0.999) {
        best = cost;
        p.rt = rt;
        p.rows = rows;
      }
    }
  }
  return p;
}

template <int MT, int RT, int NW, bool GATED, typename TO, int MODE = kFoldNone>
static void launch_skinny(const void* x, const void* w, void* y, int M, int N, int K, int ks, int rows,
                          hipStream_t stream, const SkinnyFold& fold = SkinnyFold{}) {
  // steps of loads in flight, by the registers a wave has (16 waves: 128, 8 waves: 256)
  constexpr int U = (RT + MT <= 2) ? 8 : (RT + MT <= (NW == 16 ? 4 : 7) ? 4 : 2);
  const int cap = GATED ? 16 * (RT / 2) : 16 * RT;
  if (rows <= 0 || rows > cap) rows = cap;
  const int steps = (K + 31) / 32;
  const int sps = (steps + ks - 1) / ks;
  dim3 grid((unsigned)((N + rows - 1) / rows), (unsigned)ks);
  linear_skinny_kernel<MT, RT, NW, U, GATED, TO, MODE><<<grid, NW * 64, 0, stream>>>(
      (const bf16*)x, (const bf16*)w, (TO*)y, M, N, K, sps, rows, fold);
}

// The folded forms exist for up to 16 rows and 8 waves; rt as the plan says.
template <bool GATED, typename TO, int MODE>
static bool launch_skinny_fold(int rt, int rows, const void* x, const void* w, void* y, int M, int N, int K, hipStream_t stream,
                               const SkinnyFold& fold) {
  if constexpr (!GATED) {
    if (rt == 1) { launch_skinny<1, 1, 8, false, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
    if (rt == 3) { launch_skinny<1, 3, 8, false, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
  }
  if (rt == 2) { launch_skinny<1, 2, 8, GATED, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
  if (rt == 4) { launch_skinny<1, 4, 8, GATED, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
  if (rt == 6) { launch_skinny<1, 6, 8, GATED, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
  if (rt == 8) { launch_skinny<1, 8, 8, GATED, TO, MODE>(x, w, y, M, N, K, 1, rows, stream, fold); return true; }
  return false;
}

template <int RT, int NW, bool GATED, typename TO>
static void launch_skinny_mt(int mt, const void* x, const void* w, void* y, int M, int N, int K, int ks, int rows,
                             hipStream_t stream) {
  if (mt == 1) launch_skinny<1, RT, NW, GATED, TO>(x, w, y, M, N, K, ks, rows, stream);
  else if (mt == 2) launch_skinny<2, RT, NW, GATED, TO>(x, w, y, M, N, K, ks, rows, stream);
  else if constexpr (RT <= 6) launch_skinny<4, RT, NW, GATED, TO>(x, w, y, M, N, K, ks, rows, stream);   // 33..64 rows
}

}  // namespace xi

using namespace xi;

extern "C" {

// Most rows of x the skinny kernels take.
int xi_linear_skinny_max_rows() { return 64; }

// The number of K slices xi_linear_skinny will use for these sizes (the leading dimension of
// its output when greater than 1).
int xi_linear_skinny_slices(int N, int K, int gated, int allow_split) {
  return plan_skinny(1, N, K, gated != 0, allow_split != 0).ks;
}

// The row tiles of w a workgroup takes for these sizes, and the output features it owns (they
// do not change any sum).
int xi_linear_skinny_row_tiles(int M, int N, int K, int gated, int allow_split) {
  return plan_skinny(M, N, K, gated != 0, allow_split != 0).rt;
}
int xi_linear_skinny_rows(int M, int N, int K, int gated, int allow_split) {
  return plan_skinny(M, N, K, gated != 0, allow_split != 0).rows;
}

// The product before a norm, for M <= 16 rows: resid [M, N] float32 += x [M, K] @ w [N, K]^T;
// xg [M, N] bf16 = round(resid * g) with the norm's weight g [N]; ss [M, parts] float32 = the
// sum of squares of each row of resid, in parts = xi_linear_skinny_fold_parts(M, N, K), one per
// workgroup.  The product after the norm then takes xg and ss (xi_linear_skinny_fold_in).
int xi_linear_skinny_fold_parts(int M, int N, int K) {
  const SkinnyPlan p = plan_skinny(M, N, K, false, false);
  return (N + p.rows - 1) / p.rows;
}

int xi_linear_skinny_fold_out(const void* x, const void* w, int M, int N, int K, float* resid, const float* g, void* xg,
                              float* ss, hipStream_t stream) {
  XI_CHECK(M > 0 && M <= 16 && N > 0 && K > 0 && K % 8 == 0, "linear_skinny_fold_out: bad sizes M=%d N=%d K=%d", M, N, K);
  const SkinnyPlan p = plan_skinny(M, N, K, false, false);
  SkinnyFold f{};
  f.resid = resid;
  f.g = g;
  f.xg = (bf16*)xg;
  f.ss_out = ss;
  const bool ok = launch_skinny_fold<false, bf16, kFoldOut>(p.rt, p.rows, x, w, nullptr, M, N, K, stream, f);
  XI_CHECK(ok, "linear_skinny_fold_out: no kernel of %d row tiles", p.rt);
  XI_LAUNCH_CHECK("linear_skinny_fold_out");
  return 0;
}

// The product after a norm whose first half ran in xi_linear_skinny_fold_out: xg [M, K] bf16,
// ss [M, parts] float32 (parts <= 512), y [M, N] = (xg @ w^T) * rsqrt(sum(ss[row]) / K + eps) per
// row, rounded once; gated as in xi_linear_skinny (then y is bfloat16).
int xi_linear_skinny_fold_in(const void* xg, const void* w, void* y, int M, int N, int K, int out_dtype, int gated,
                             const float* ss, int parts, float eps, hipStream_t stream) {
  XI_CHECK(M > 0 && M <= 16 && N > 0 && K > 0 && K % 8 == 0, "linear_skinny_fold_in: bad sizes M=%d N=%d K=%d", M, N, K);
  XI_CHECK(parts > 0 && parts <= 512, "linear_skinny_fold_in: %d parts of a row's sum of squares (at most 512)", parts);
  XI_CHECK(out_dtype == kBF16 || (out_dtype == kF32 && !gated), "linear_skinny_fold_in: output dtype %d", out_dtype);
  const SkinnyPlan p = plan_skinny(M, N, K, gated != 0, false);
  SkinnyFold f{};
  f.ss_in = ss;
  f.parts = parts;
  f.eps = eps;
  f.inv_h = 1.f / (float)K;
  bool ok;
  if (gated) ok = launch_skinny_fold<true, bf16, kFoldIn>(p.rt, p.rows, xg, w, y, M, N, K, stream, f);
  else if (out_dtype == kBF16) ok = launch_skinny_fold<false, bf16, kFoldIn>(p.rt, p.rows, xg, w, y, M, N, K, stream, f);
  else ok = launch_skinny_fold<false, float, kFoldIn>(p.rt, p.rows, xg, w, y, M, N, K, stream, f);
  XI_CHECK(ok, "linear_skinny_fold_in: no kernel of %d row tiles", p.rt);
  XI_LAUNCH_CHECK("linear_skinny_fold_in");
  return 0;
}

// x [M, K] bf16, w [N, K] bf16 -> y [M, N] in out_dtype (bf16 or float32); with
// allow_split and xi_linear_skinny_slices(...) = KS > 1, y is float32 [KS, M, N] partial sums.
// gated != 0: w is [2N, K] and y [M, N] = silu(x @ w[:N]^T) * (x @ w[N:]^T), bfloat16.
// force_rt / force_nw: 0 = chosen from the sizes; other values select a shape (for measurements
// and tests; nw * rt must not exceed 32).
int xi_linear_skinny(const void* x, const void* w, void* y, int M, int N, int K, int out_dtype, int gated,
                     int allow_split, int force_rt, int force_nw, hipStream_t stream) {
  XI_CHECK(M >= 0 && N > 0 && K > 0, "linear_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  XI_CHECK(M <= 64, "linear_skinny: %d rows exceed 64 (use the library product)", M);
  XI_CHECK(K % 8 == 0, "linear_skinny: K=%d must be a multiple of 8", K);
  XI_CHECK(out_dtype == kBF16 || out_dtype == kF32, "linear_skinny: unknown output dtype %d", out_dtype);
  if (M == 0) return 0;
  SkinnyPlan p = plan_skinny(M, N, K, gated != 0, allow_split != 0);
  XI_CHECK(p.ks == 1 || out_dtype == kF32, "linear_skinny: partial sums of %d slices must be float32", p.ks);
  XI_CHECK(!gated || out_dtype == kBF16, "linear_skinny: the gated form writes bfloat16");
  if (force_nw) p.nw = force_nw;
  if (force_rt) {
    p.rt = force_rt;
    p.rows = 0;          // whole tiles
  }
  XI_CHECK(p.nw == 8 || p.nw == 16, "linear_skinny: %d waves (8 or 16)", p.nw);
  const int mt = (M + 15) / 16;
  XI_CHECK(skinny_shape_ok(p.rt, p.nw, mt, gated != 0), "linear_skinny: no kernel of %d row tiles, %d waves for %d rows%s",
           p.rt, p.nw, M, gated ? " (gated)" : "");
#define XI_SK_PLAIN(RT, NW)                                                       \
  do {                                                                            \
    if (out_dtype == kBF16)                                                       \
      launch_skinny_mt<RT, NW, false, bf16>(mt, x, w, y, M, N, K, p.ks, p.rows, stream);  \
    else                                                                          \
      launch_skinny_mt<RT, NW, false, float>(mt, x, w, y, M, N, K, p.ks, p.rows, stream); \
  } while (0)
#define XI_SK_GATED(RT, NW) launch_skinny_mt<RT, NW, true, bf16>(mt, x, w, y, M, N, K, p.ks, p.rows, stream)
  if (gated) {
    if (p.nw == 16) XI_SK_GATED(2, 16);
    else if (p.rt == 2) XI_SK_GATED(2, 8);
    else if (p.rt == 4) XI_SK_GATED(4, 8);
    else if (p.rt == 6) XI_SK_GATED(6, 8);
    else XI_SK_GATED(8, 8);
  } else if (p.nw == 16) {
    if (p.rt == 1) XI_SK_PLAIN(1, 16);
    else XI_SK_PLAIN(2, 16);
  } else {
    if (p.rt == 1) XI_SK_PLAIN(1, 8);
    else if (p.rt == 2) XI_SK_PLAIN(2, 8);
    else if (p.rt == 3) XI_SK_PLAIN(3, 8);
    else if (p.rt == 4) XI_SK_PLAIN(4, 8);
    else if (p.rt == 6) XI_SK_PLAIN(6, 8);
    else XI_SK_PLAIN(8, 8);
  }
#undef XI_SK_PLAIN
#undef XI_SK_GATED
  XI_LAUNCH_CHECK("linear_skinny");
  return 0;
}

}  // extern "C"
