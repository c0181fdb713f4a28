// y[M,N] = x[M,K] @ w[N,K]^T in bfloat16 for decode batches of 17 to 128 rows and narrow
// outputs (o and down projections): still bound by the one pass over w, but with so many rows
// that a workgroup has to own many output features per read of x, or the reads of x from L2
// cost more than the stream of w.  The vendor library has too few tiles for these shapes
// (N = 4096 at 128 rows is 32 tiles for 256 compute units) and runs them at a fifth to a third
// of the memory bandwidth.  Measured on MI355X (N = 5120, K = 17408, 178 MB of w, 29 us at the
// 6.2 TB/s a streaming read reaches): 33 us at 17 rows, 36 at 64, 45 at 128, against 124 to
// 149 us for the library; what is left above the stream is the read of x from L2, M / 128 of
// the bytes of w.
//
// A workgroup of four waves owns 128 output features, all rows of x (up to 128) and one of KS
// slices of K, so that tiles x slices fill the compute units; the slices' float32 partial sums
// [KS, M, N] are added in slice order by the consumer (the fused add + RMSNorm).  It walks its
// slice in tiles of 64: all 256 threads copy the w tile [128 features, 64] and the x tile
// [128 rows, 64] from memory into registers, two tiles ahead, and from there into LDS
// (double buffered: one barrier a tile); a wave multiplies its quarter, 64 features by 64 rows,
// as 4 x 4 v_mfma_f32_16x16x32_bf16 tiles per 32-wide k step (A = 16 rows of w, B = 16 rows of
// x, as in linear_skinny.hip).  LDS rows are padded by 16 bytes so that the 16 lanes that read
// one operand together fall into 16 different 16-byte bank groups.
//
// Workgroup b takes slice b % KS: with 8 slices on 8 XCDs (workgroups go round the XCDs) each
// L2 holds one slice of x.  An output element's value depends on (N, K) alone (they fix KS):
// never on M or on what else is in the batch.
//
// GATED: w is [2N, K] = [gate; up] (the feed-forward's first product, which is wide: no slices);
// a workgroup owns R <= 64 features n0 .. n0 + R - 1 (any R, so that the grid is a multiple of
// the compute units), its tile holds their gate rows in rows 0 .. 63 and their up rows in rows
// 64 .. 127, a wave multiplies 16-feature tiles of both, and stores silu(gate) * up in bfloat16:
// one pass over w at any M up to 128, where the streaming kernel's workgroups (16 to 50
// features) re-read x from L2 more the more rows there are.  FOLD: x is the first half of a
// folded RMSNorm (see linear_skinny.hip): the rows of the product are multiplied by
// rsqrt(sum of the row's parts / K + eps) before the activation.  WR = 8: a tile of 256 rows of w,
// R <= 128 features a workgroup (up to 64 rows of x): where 64 features make two rounds of
// workgroups (intermediate sizes above 16,384) one round of twice the features reads x from L2
// half as often; at 17 to 64 rows, where x is as many bytes as a workgroup's share of w.
//
// Reference call site: candle matmul in /root/reference/src/models/layers/linear.rs:76-124
// (vendor BLAS).
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kMidRows = 128;          // rows of x a workgroup takes: all of them
constexpr int kMidFeatures = 128;      // rows of w in a workgroup's tile
constexpr int kMidK = 64;              // k per tile
constexpr int kMidLdsRow = kMidK + 8;  // elements of a row in LDS
constexpr int kMidDepth = 2;           // tiles whose loads are in flight (the default; measured: more gain nothing)
constexpr int kMidTile = 128 * kMidLdsRow;   // elements of one operand's tile in LDS
constexpr size_t kMidLdsBytes = 2 * 2 * (size_t)kMidTile * sizeof(bf16) + 16 * sizeof(float);
constexpr size_t kMidWideLdsBytes = 2 * 3 * (size_t)kMidTile * sizeof(bf16) + 16 * sizeof(float);   // WR = 8
constexpr int kMidSsLoads = 32;        // 16 threads x 32 loads: up to 512 parts of a row's sum of squares

struct MidFold {
  const float* ss_in;   // [M, parts] parts of each row's sum of squares
  int parts;
  float eps;
  float inv_h;          // 1 / length of the normed rows
};

// D: tiles whose loads are in flight.  FULL: up to 128 rows of x, the four waves take a quarter
// of the tile each (64 rows of w by 64 rows of x); else up to 16 * TJ <= 64 rows of x and a wave
// takes a quarter of the rows of w (32) by all rows of x.  GATED, FOLD: see the head of the file.
template <int D, int TJ, bool FULL, bool GATED, bool FOLD, int WR = 4>
__global__ __launch_bounds__(256, 1) void linear_mid_kernel(const bf16* __restrict__ x,
                                                            const bf16* __restrict__ w, void* __restrict__ yv,
                                                            int M, int N, int K, int ks, size_t slice_stride,
                                                            int R, int rotate, MidFold fold) {
  static_assert(!FULL || TJ == 4, "the full form multiplies 64 rows of x per wave");
  static_assert(!FOLD || (GATED && !FULL && TJ == 1), "a folded norm: the gated form, up to 16 rows");
  static_assert(WR == 4 || (WR == 8 && GATED && !FULL && !FOLD), "the tile of 256 rows of w: the gated form, up to 64 rows of x");
  constexpr int WROWS = 32 * WR;                      // rows of the w tile
  constexpr int HALF = WROWS / 2;                     // GATED: so many gate rows, then as many up rows
  constexpr int WT = WROWS * kMidLdsRow;              // elements of the w tile in LDS (the x tile: kMidTile)
  extern __shared__ __align__(16) unsigned char mid_smem[];
  bf16* lds = reinterpret_cast<bf16*>(mid_smem);   // [buffer][w tile [WROWS] | x tile [128]][kMidLdsRow]
  float* inv_s = reinterpret_cast<float*>(mid_smem + 2 * (size_t)(WT + kMidTile) * sizeof(bf16));   // [16]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  constexpr int TI = FULL ? 4 : WR / 2;               // 16-row tiles of w a wave multiplies
  constexpr int TG = GATED ? TI / 2 : TI;             // of them gate tiles (the others: their up tiles)
  constexpr int XI = FULL ? 4 : (TJ == 4 ? 2 : 1);    // 32-row groups of x that are copied
  const int wf = FULL ? (wave & 1) : wave;            // which of the wave's shares of the features,
  const int wt = FULL ? (wave >> 1) : 0;              // of the rows of x (64 * wt on)
  const int slice = blockIdx.x % ks, tile = blockIdx.x / ks;
  const int n0 = tile * R;
  const int n_last = (n0 + R < N ? n0 + R : N) - 1;   // the workgroup's last feature
  // the k tiles of this slice: K / 64 tiles dealt out as evenly as they go
  const int kt_total = K / kMidK;
  const int base = kt_total / ks, rem = kt_total % ks;
  const int kt0 = slice * base + (slice < rem ? slice : rem);
  const int nkt = base + (slice < rem ? 1 : 0);
  // Workgroups start at different tiles of their slice and wrap around, so that they do not all
  // ask for the same offset of their rows of w at the same time; where a workgroup starts
  // depends on its features alone, so an output element's sum has one order whatever M is.
  const int start = (int)(((long long)tile * rotate) % nkt);

  // FOLD: 16 threads per row add up the parts of its sum of squares; the loads start now
  float ss_mine[FOLD ? kMidSsLoads : 1];
  if constexpr (FOLD) {
    const int token = tid >> 4, sub = tid & 15;
#pragma unroll
    for (int i = 0; i < kMidSsLoads; ++i) {
      const int p = sub + 16 * i;
      ss_mine[i] = (token < M && p < fold.parts) ? fold.ss_in[(size_t)token * fold.parts + p] : 0.f;
    }
  }

  // ---- copying: a tile is 128 rows (of w: WROWS) of 8 16-byte chunks; thread t moves chunk t % 8 of rows
  // t / 8 + 32 i.  Row q of the w tile is feature n0 + q (GATED: the gate row of feature
  // n0 + q % HALF for q < HALF, its up row for q >= HALF); rows past the workgroup's last feature read
  // that feature's row again and rows of x past M row M - 1 (the same address many times in one
  // instruction costs one access); their results are dropped.  No load is conditional, so the
  // counter of loads in flight is exact and only the tile that is needed is waited for.
  const int srow = tid >> 3, skc = tid & 7;
  const bf16* wsrc[WR];
  const bf16* xsrc[XI];
#pragma unroll
  for (int i = 0; i < WR; ++i) {
    const int row = srow + 32 * i;
    int n = n0 + (GATED ? (row & (HALF - 1)) : row);
    n = n < n_last ? n : n_last;
    if (GATED && row >= HALF) n += N;
    wsrc[i] = w + (size_t)n * K + (size_t)kt0 * kMidK + 8 * skc;
  }
#pragma unroll
  for (int i = 0; i < XI; ++i) {
    const int row = srow + 32 * i;
    xsrc[i] = x + (size_t)(row < M ? row : M - 1) * K + (size_t)kt0 * kMidK + 8 * skc;
  }
  const int sdst = srow * kMidLdsRow + 8 * skc;
  bf16x8 wr[D][WR], xr[D][XI];

  // a wave whose rows of x lie past M, or whose features past the workgroup's, has nothing to do
  const int wave_row0 = GATED ? 16 * TG * wf : 16 * TI * wf;     // its first feature within the workgroup
  const bool active = __builtin_amdgcn_readfirstlane((64 * wt < M && n0 + wave_row0 <= n_last) ? 1 : 0) != 0;
  f32x4 acc[TI][TJ];
#pragma unroll
  for (int ti = 0; ti < TI; ++ti)
#pragma unroll
    for (int tj = 0; tj < TJ; ++tj) acc[ti][tj] = f32x4{0.f, 0.f, 0.f, 0.f};

#define XI_MID_ISSUE(slot, t)                                                         \
  do {                                                                                \
    int tt_ = (t) + start;                                                            \
    tt_ = tt_ >= nkt ? tt_ - nkt : tt_;                                               \
    _Pragma("unroll") for (int i = 0; i < WR; ++i)                                    \
      wr[slot][i] = *reinterpret_cast<const bf16x8*>(wsrc[i] + (size_t)tt_ * kMidK);  \
    _Pragma("unroll") for (int i = 0; i < XI; ++i)                                    \
      xr[slot][i] = *reinterpret_cast<const bf16x8*>(xsrc[i] + (size_t)tt_ * kMidK);  \
  } while (0)

  // Every copy is issued whether or not its tile exists (past the slice's end the last tile is
  // read again, from cache, and dropped): with a fixed number of loads between a tile's loads
  // and its use, the wait before the use leaves exactly the younger tiles in flight.
  const int last = nkt - 1;
#pragma unroll
  for (int s = 0; s < D; ++s) XI_MID_ISSUE(s, s < last ? s : last);

  // One tile: registers of slot s to LDS, the slot loaded again D tiles ahead, barrier,
  // products.  One barrier a tile is enough: whoever writes this buffer again, two tiles on, has
  // passed the next tile's barrier, which every thread reaches only after these products.
  // Row of the w tile of the wave's tile ti: its features' rows; GATED: gate tiles first, then
  // the up tiles of the same features, HALF rows further.
  int buf = 0;
#define XI_MID_WROW(ti) (GATED ? (((ti) / TG) * HALF + wave_row0 + 16 * ((ti) % TG)) : (wave_row0 + 16 * (ti)))
#define XI_MID_TILE(s, t)                                                                                 \
  do {                                                                                                    \
    bf16* Ws = lds + buf * (WT + kMidTile);                                                               \
    bf16* Xs = Ws + WT;                                                                                   \
    _Pragma("unroll") for (int i = 0; i < WR; ++i)                                                        \
      *reinterpret_cast<bf16x8*>(Ws + sdst + 32 * i * kMidLdsRow) = wr[s][i];                             \
    _Pragma("unroll") for (int i = 0; i < XI; ++i)                                                        \
      *reinterpret_cast<bf16x8*>(Xs + sdst + 32 * i * kMidLdsRow) = xr[s][i];                             \
    XI_MID_ISSUE(s, (t) + D < last ? (t) + D : last);                                                     \
    __syncthreads();                                                                                      \
    if (active) {                                                                                         \
      _Pragma("unroll") for (int kk = 0; kk < kMidK / 32; ++kk) {                                         \
        bf16x8 a[TI], b[TJ];                                                                              \
        _Pragma("unroll") for (int ti = 0; ti < TI; ++ti) a[ti] = *reinterpret_cast<const bf16x8*>(       \
            Ws + (XI_MID_WROW(ti) + r) * kMidLdsRow + 32 * kk + 8 * j);                                   \
        _Pragma("unroll") for (int tj = 0; tj < TJ; ++tj) b[tj] = *reinterpret_cast<const bf16x8*>(       \
            Xs + (64 * wt + 16 * tj + r) * kMidLdsRow + 32 * kk + 8 * j);                                 \
        _Pragma("unroll") for (int ti = 0; ti < TI; ++ti)                                                 \
          _Pragma("unroll") for (int tj = 0; tj < TJ; ++tj)                                               \
            acc[ti][tj] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[ti], b[tj], acc[ti][tj], 0, 0, 0);    \
      }                                                                                                   \
    }                                                                                                     \
    buf ^= 1;                                                                                             \
  } while (0)

  // whole rotations of the slots in a loop without exits inside, then the tiles that are left
  int t0 = 0;
  for (; t0 + D <= nkt; t0 += D) {
#pragma unroll
    for (int s = 0; s < D; ++s) XI_MID_TILE(s, t0 + s);
  }
#pragma unroll
  for (int s = 0; s < D - 1; ++s)
    if (t0 + s < nkt) XI_MID_TILE(s, t0 + s);     // the same for every thread
#undef XI_MID_TILE
#undef XI_MID_ISSUE

  if constexpr (FOLD) {
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kMidSsLoads; ++i) t += ss_mine[i];
    t += lane_xor<8>(t);
    t += lane_xor<4>(t);
    t += lane_xor<2>(t);
    t += lane_xor<1>(t);
    if ((tid & 15) == 0) inv_s[tid >> 4] = rsqrtf(t * fold.inv_h + fold.eps);
    __syncthreads();
  }
  if (!active) return;

  // a lane's 4 values of a tile: row 16 tj + r of x, features 4 j .. 4 j + 3 of the tile
  if constexpr (GATED) {
    bf16* y = reinterpret_cast<bf16*>(yv);
#pragma unroll
    for (int tj = 0; tj < TJ; ++tj) {
      const int token = 64 * wt + 16 * tj + r;
      if (token >= M) continue;
      const float inv = FOLD ? inv_s[token] : 1.f;
#pragma unroll
      for (int ti = 0; ti < TG; ++ti) {
        const int f = n0 + wave_row0 + 16 * ti + 4 * j;
        bf16* dst = y + (size_t)token * N + f;
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (f + i <= n_last) {
            const float g = acc[ti][tj][i] * inv, u = acc[ti + TG][tj][i] * inv;
            dst[i] = from_float<bf16>(g / (1.f + __expf(-g)) * u);
          }
      }
    }
  } else {
    float* ys = reinterpret_cast<float*>(yv) + (size_t)slice * slice_stride;
    const bool vec = (N & 3) == 0;
#pragma unroll
    for (int tj = 0; tj < TJ; ++tj) {
      const int token = 64 * wt + 16 * tj + r;
      if (token >= M) continue;
#pragma unroll
      for (int ti = 0; ti < TI; ++ti) {
        const int f = n0 + wave_row0 + 16 * ti + 4 * j;
        float* dst = ys + (size_t)token * N + f;
        if (vec && f + 3 <= n_last) {
          *reinterpret_cast<f32x4*>(dst) = acc[ti][tj];
        } else {
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (f + i <= n_last) dst[i] = acc[ti][tj][i];
        }
      }
    }
  }
}
#undef XI_MID_WROW

// Slices of K for an output of N features: tiles x slices fill the 256 compute units once; a
// slice keeps at least 4 tiles of 64.  It depends on (N, K) alone.
static int mid_slices(int N, int K) {
  const int tiles = (N + kMidFeatures - 1) / kMidFeatures;
  const int kt = K / kMidK;
  int ks = 256 / tiles;
  if (ks > 16) ks = 16;
  while (ks > 1 && kt / ks < 4) --ks;
  return ks < 1 ? 1 : ks;
}

// Features a workgroup of the gated form owns (at most `most`: 64, or 128 for the tile of 256
// rows of w): the fewest workgroups that are a multiple of the 256 compute units, or failing that
// (N < 256 or so) of 64 features each.
static int mid_gated_features(int N, int most = 64) {
  for (int waves = 1; waves <= 64; ++waves) {
    const int wgs = 256 * waves;
    const int rr = (N + wgs - 1) / wgs;
    if (rr <= most) return rr < 16 ? 16 : rr;     // a narrow output: whole 16-feature tiles
  }
  return 64;
}

template <typename Kern>
static int mid_lds(Kern kern, bool* done, size_t bytes = kMidLdsBytes) {
  if (*done) return 0;
  hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
  XI_CHECK(e == hipSuccess, "linear_mid: cannot get %zu bytes of LDS: %s", bytes, hipGetErrorString(e));
  *done = true;
  return 0;
}

}  // namespace xi

using namespace xi;

extern "C" {

int xi_linear_mid_max_rows() { return 2 * kMidRows; }

// 0 if the sizes are not taken (the caller then uses another product).
int xi_linear_mid_slices(int N, int K) {
  if (N < 1 || K < kMidK || K % kMidK) return 0;
  return mid_slices(N, K);
}

// Features per workgroup of the gated form for an output of N features (w is [2N, K]) at M rows.
// From 17 to 64 rows a workgroup takes up to 128 features where that saves a round of workgroups.
int xi_linear_mid_gated_features(int N, int M) {
  if (N < 1) return 0;
  const int r = mid_gated_features(N);
  if (M > 16 && M <= 64) {
    const int wide = mid_gated_features(N, 128);
    if (wide > 64 && (N + wide - 1) / wide < (N + r - 1) / r) return wide;
  }
  return r;
}

// y: float32 [slices, M, N] with slices = xi_linear_mid_slices(N, K).  Up to 256 rows: blocks of
// 128 rows are launched one after the other (the second pass over w comes in part from the
// last level cache).  depth: tiles of loads in flight, 0 = the default (the result does not
// depend on it).
int xi_linear_mid(const void* x, const void* w, float* y, int M, int N, int K, int depth, int rotate,
                  hipStream_t stream) {
  XI_CHECK(M >= 1 && M <= 2 * kMidRows, "linear_mid: M=%d must be 1..%d", M, 2 * kMidRows);
  XI_CHECK(N >= 1 && K >= kMidK && K % kMidK == 0, "linear_mid: N=%d, K=%d (a multiple of %d) are not taken", N, K, kMidK);
  XI_CHECK(((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) % 16 == 0, "linear_mid: operands must be 16-byte aligned");
  XI_CHECK(rotate >= 0, "linear_mid: rotate=%d", rotate);
  const int ks = mid_slices(N, K);
  const long long tiles = (N + kMidFeatures - 1) / kMidFeatures;
  XI_CHECK(ks >= 1 && ks <= K / kMidK, "linear_mid: %d slices for K=%d", ks, K);
  XI_CHECK(tiles * ks < (1ll << 31), "linear_mid: too many workgroups");
  if (depth == 0) depth = kMidDepth;
  const MidFold none{nullptr, 0, 0.f, 0.f};
#define XI_MID(D, TJ, FULL)                                                                                   \
  do {                                                                                                        \
    static bool lds_set = false;                                                                              \
    if (mid_lds(linear_mid_kernel<D, TJ, FULL, false, false>, &lds_set)) return 1;                            \
    linear_mid_kernel<D, TJ, FULL, false, false><<<(unsigned)(tiles * ks), 256, kMidLdsBytes, stream>>>(      \
        (const bf16*)x + (size_t)row0 * K, (const bf16*)w, y + (size_t)row0 * N, rows, N, K, ks,              \
        (size_t)M * N, kMidFeatures, rotate, none);                                                           \
  } while (0)
#define XI_MID_D(D)                                        \
  do {                                                     \
    for (int row0 = 0; row0 < M; row0 += kMidRows) {       \
      const int rows = M - row0 < kMidRows ? M - row0 : kMidRows; \
      if (rows <= 64) XI_MID(D, 4, false);                 \
      else XI_MID(D, 4, true);                             \
    }                                                      \
  } while (0)
  if (depth == 2) XI_MID_D(2);
  else if (depth == 3) XI_MID_D(3);
  else if (depth == 4) XI_MID_D(4);
  else XI_CHECK(false, "linear_mid: no kernel with %d tiles in flight", depth);
#undef XI_MID_D
#undef XI_MID
  XI_LAUNCH_CHECK("linear_mid");
  return 0;
}

// y [M, N] bfloat16 = silu(x @ gate^T) * (x @ up^T) with w = [gate; up] [2N, K], M <= 128.
// ss (or null): x is the first half of a folded RMSNorm, ss [M, parts] float32 the parts of its
// rows' sums of squares (M <= 16, parts <= 512): rows are scaled by rsqrt(sum / K + eps).
int xi_linear_mid_gated(const void* x, const void* w, void* y, int M, int N, int K, const float* ss, int parts,
                        float eps, int rotate, int features, hipStream_t stream) {
  XI_CHECK(M >= 1 && M <= kMidRows, "linear_mid_gated: M=%d must be 1..%d", M, kMidRows);
  XI_CHECK(N >= 1 && K >= kMidK && K % kMidK == 0, "linear_mid_gated: N=%d, K=%d (a multiple of %d) are not taken", N,
           K, kMidK);
  XI_CHECK(((uintptr_t)x | (uintptr_t)w) % 16 == 0, "linear_mid_gated: operands must be 16-byte aligned");
  XI_CHECK(rotate >= 0, "linear_mid_gated: rotate=%d", rotate);
  XI_CHECK(ss == nullptr || (M <= 16 && parts >= 1 && parts <= 16 * kMidSsLoads),
           "linear_mid_gated: a folded norm takes up to 16 rows and %d parts (M=%d, parts=%d)", 16 * kMidSsLoads, M, parts);
  const int R = features > 0 ? features : xi_linear_mid_gated_features(N, M);     // features: an override, for measurements
  const long long wgs = (N + R - 1) / R;
  XI_CHECK(R >= 1 && R <= 128 && wgs < (1ll << 31), "linear_mid_gated: %d features per workgroup", R);
  XI_CHECK(R <= 64 || (M <= 64 && ss == nullptr), "linear_mid_gated: %d features per workgroup are taken up to 64 rows, without a folded norm", R);
  const MidFold fold{ss, parts, eps, 1.f / (float)K};
  if (R > 64) {
#define XI_MIDW(TJ)                                                                                                     \
  do {                                                                                                                  \
    static bool lds_set = false;                                                                                        \
    if (mid_lds(linear_mid_kernel<kMidDepth, TJ, false, true, false, 8>, &lds_set, kMidWideLdsBytes)) return 1;         \
    linear_mid_kernel<kMidDepth, TJ, false, true, false, 8><<<(unsigned)wgs, 256, kMidWideLdsBytes, stream>>>(          \
        (const bf16*)x, (const bf16*)w, y, M, N, K, 1, 0, R, rotate, fold);                                             \
  } while (0)
    if (M <= 16) XI_MIDW(1);
    else if (M <= 32) XI_MIDW(2);
    else XI_MIDW(4);
#undef XI_MIDW
    XI_LAUNCH_CHECK("linear_mid_gated");
    return 0;
  }
#define XI_MIDG(TJ, FULL, FOLD)                                                                               \
  do {                                                                                                        \
    static bool lds_set = false;                                                                              \
    if (mid_lds(linear_mid_kernel<kMidDepth, TJ, FULL, true, FOLD>, &lds_set)) return 1;                      \
    linear_mid_kernel<kMidDepth, TJ, FULL, true, FOLD><<<(unsigned)wgs, 256, kMidLdsBytes, stream>>>(         \
        (const bf16*)x, (const bf16*)w, y, M, N, K, 1, 0, R, rotate, fold);                                   \
  } while (0)
  if (ss != nullptr) XI_MIDG(1, false, true);
  else if (M <= 16) XI_MIDG(1, false, false);
  else if (M <= 32) XI_MIDG(2, false, false);
  else if (M <= 64) XI_MIDG(4, false, false);
  else XI_MIDG(4, true, false);
#undef XI_MIDG
  XI_LAUNCH_CHECK("linear_mid_gated");
  return 0;
}

}  // extern "C"
