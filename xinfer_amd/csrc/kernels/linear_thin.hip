// y[M,N] = x[M,K] @ w[N,K]^T in bfloat16 for up to 16 rows (a decode step of few requests) where
// every workgroup has to own few output features so that the whole chip works on a narrow
// output without slices of K: the products around a folded RMSNorm (linear_skinny.hip describes
// the fold), which need whole sums.  The streaming kernel there loads 16 rows of w by 64 bytes
// per instruction, and its counters show the texture addresser stalled half of the time; this
// kernel asks for the same bytes as whole lines.
//
// A workgroup of four waves owns R <= 32 features (R from N alone, so that the workgroups are a
// multiple of the 256 compute units) and all of K.  It walks K in tiles of 256: all 256 threads
// copy the w tile [32 rows, 512 bytes each: 32 lanes a row] and the x tile [4, 8 or 16 rows] from
// memory into registers, two tiles ahead, and from there into LDS (double buffered, one barrier
// a tile); wave v multiplies k steps 2v and 2v+1 of the tile's eight (v_mfma_f32_16x16x32_bf16,
// A = 16 rows of w, B = the 16 rows of x), two tiles of 16 features each.  Workgroups of up to
// 16 features take tiles of [16 rows, 512 k] instead: the same bytes a tile, no rows that
// nobody multiplies, half the barriers.  At the end the four
// waves' sums are added through LDS in wave order and stored: plain (MODE 0), adding into the
// float32 residual stream and handing on round(stream * g) and the rows' sums of squares (MODE
// 1), or scaling the rows by rsqrt(sum of the parts / K + eps) (MODE 2).
//
// Workgroup b starts b * rotate tiles into K and wraps around (see linear_mid.hip).  An output
// element's value depends on (N, K) alone, never on M or on what else is in the batch.
//
// Reference call site: candle matmul in /root/reference/src/models/layers/linear.rs:76-124.
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kThinRows = 16;            // rows of x
constexpr int kThinFeatures = 32;        // most rows of w in a workgroup's tile
constexpr int kThinK = 256;              // k per tile of 32 rows of w (a tile of 16 rows takes 512: the same bytes)
constexpr int kThinDepth = 2;            // tiles whose loads are in flight
constexpr int kThinSsLoads = 32;         // 16 threads x 32 loads: up to 512 parts of a row's sum of squares
constexpr size_t thin_lds_bytes(int tr) {     // two buffers of a w tile and an x tile, rows padded by 8 elements
  return 2 * (size_t)(tr + kThinRows) * (8192 / tr + 8) * sizeof(bf16);
}

struct ThinFold {
  float* resid;         // MODE 1: [M, N] float32, updated in place
  const float* g;       // MODE 1: [N] weight of the norm that follows
  bf16* xg;             // MODE 1: [M, N]
  float* ss_out;        // MODE 1: [M, gridDim.x]
  const float* ss_in;   // MODE 2: [M, parts]
  int parts;            // MODE 2
  float eps;            // MODE 2
  float inv_h;          // MODE 2: 1 / length of the normed rows
};

// TR: rows of w in a tile, 32 or 16 (for workgroups of up to 16 features: no rows are copied
// that nobody multiplies); a tile holds 8192 / TR of k.  XR: rows of x in a tile, the power of
// two from M up that the copying takes (a workgroup reads all of x, as many bytes per row as of
// a row of w, so rows that are not there cost as much as features); the product's rows past XR
// repeat earlier ones and are dropped.
template <int MODE, typename TO, int TR, int XR>
__global__ __launch_bounds__(256) void linear_thin_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                          TO* __restrict__ y, int M, int N, int K, int R, int rotate,
                                                          ThinFold fold) {
  constexpr int D = kThinDepth;
  constexpr int BK = 8192 / TR;              // k per tile
  constexpr int LROW = BK + 8;               // elements of a row in LDS
  constexpr int CPR = BK / 8;                // 16-byte chunks of a row
  constexpr int RPP = 256 / CPR;             // rows the 256 threads copy at once
  constexpr int WP = TR / RPP, XP = XR / RPP;
  static_assert(XR % RPP == 0 && XP >= 1, "rows of x in a tile");     // copies of a thread per tile of w, of x
  constexpr int RT = TR / 16;                // 16-feature tiles
  constexpr int SPW = BK / 32 / 4;           // 32-wide k steps of a tile that a wave multiplies
  constexpr int STAGE = (TR + XR) * LROW;         // elements of one buffer
  extern __shared__ __align__(16) unsigned char thin_smem[];
  bf16* lds = reinterpret_cast<bf16*>(thin_smem);        // [buffer][w tile TR rows | x tile 16 rows][LROW]
  __shared__ __align__(16) float red[4 * RT * 256];      // [wave][feature tile][lane * 4 + i]
  __shared__ float side[MODE == 1 ? kThinRows * TR : kThinRows];   // squares [row][feature], or 1/rms [row]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int n0 = blockIdx.x * R;
  const int n_last = (n0 + R < N ? n0 + R : N) - 1;
  const int nkt = K / BK;
  const int start = (int)(((long long)blockIdx.x * rotate) % nkt);

  // MODE 2: 16 threads per row add up the parts of its sum of squares; the loads start now
  float ss_mine[MODE == 2 ? kThinSsLoads : 1];
  if constexpr (MODE == 2) {
    const int token = tid >> 4, sub = tid & 15;
#pragma unroll
    for (int i = 0; i < kThinSsLoads; ++i) {
      const int p = sub + 16 * i;
      ss_mine[i] = (token < M && p < fold.parts) ? fold.ss_in[(size_t)token * fold.parts + p] : 0.f;
    }
  }

  // ---- copying: a row of a tile is CPR 16-byte chunks; thread t moves chunk t % CPR of rows
  // t / CPR + RPP i of w (i < WP) and of x (i < XP).  Rows past the workgroup's last feature
  // read that feature's row again, rows of x past M row M - 1; no load is conditional.
  const int srow = tid / CPR, skc = tid % CPR;
  const bf16* wsrc[WP];
  const bf16* xsrc[XP];
#pragma unroll
  for (int i = 0; i < WP; ++i) {
    int n = n0 + srow + RPP * i;
    n = n < n_last ? n : n_last;
    wsrc[i] = w + (size_t)n * K + 8 * skc;
  }
#pragma unroll
  for (int i = 0; i < XP; ++i) {
    const int row = srow + RPP * i;
    xsrc[i] = x + (size_t)(row < M ? row : M - 1) * K + 8 * skc;
  }
  const int sdst = srow * LROW + 8 * skc;
  bf16x8 wr[D][WP], xr[D][XP];
  f32x4 acc[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};

#define XI_THIN_ISSUE(slot, t)                                                           \
  do {                                                                                   \
    int tt_ = (t) + start;                                                               \
    tt_ = tt_ >= nkt ? tt_ - nkt : tt_;                                                  \
    _Pragma("unroll") for (int i = 0; i < WP; ++i)                                       \
      wr[slot][i] = *reinterpret_cast<const bf16x8*>(wsrc[i] + (size_t)tt_ * BK);        \
    _Pragma("unroll") for (int i = 0; i < XP; ++i)                                       \
      xr[slot][i] = *reinterpret_cast<const bf16x8*>(xsrc[i] + (size_t)tt_ * BK);        \
  } while (0)

  // every copy is issued whether or not its tile exists (past the end the last tile is read
  // again and dropped), so that the wait before a tile's use leaves the younger loads in flight
  const int last = nkt - 1;
#pragma unroll
  for (int s = 0; s < D; ++s) XI_THIN_ISSUE(s, s < last ? s : last);

  int buf = 0;
#define XI_THIN_TILE(s, t)                                                                                \
  do {                                                                                                    \
    bf16* Ws = lds + buf * STAGE;                                                                         \
    bf16* Xs = Ws + TR * LROW;                                                                            \
    _Pragma("unroll") for (int i = 0; i < WP; ++i)                                                        \
      *reinterpret_cast<bf16x8*>(Ws + sdst + RPP * i * LROW) = wr[s][i];                                  \
    _Pragma("unroll") for (int i = 0; i < XP; ++i)                                                        \
      *reinterpret_cast<bf16x8*>(Xs + sdst + RPP * i * LROW) = xr[s][i];                                  \
    XI_THIN_ISSUE(s, (t) + D < last ? (t) + D : last);                                                    \
    __syncthreads();                                                                                      \
    _Pragma("unroll") for (int kk = 0; kk < SPW; ++kk) {                                                  \
      const int col = 32 * (SPW * wave + kk) + 8 * j;                                                     \
      const bf16x8 b = *reinterpret_cast<const bf16x8*>(Xs + (r & (XR - 1)) * LROW + col);                             \
      _Pragma("unroll") for (int t_ = 0; t_ < RT; ++t_) {                                                 \
        const bf16x8 a = *reinterpret_cast<const bf16x8*>(Ws + (16 * t_ + r) * LROW + col);               \
        acc[t_] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[t_], 0, 0, 0);                        \
      }                                                                                                   \
    }                                                                                                     \
    buf ^= 1;                                                                                             \
  } while (0)

  // whole rotations of the slots in a loop without exits inside, then the tiles that are left;
  // one barrier a tile is enough (see linear_mid.hip)
  int t0 = 0;
  for (; t0 + D <= nkt; t0 += D) {
#pragma unroll
    for (int s = 0; s < D; ++s) XI_THIN_TILE(s, t0 + s);
  }
#pragma unroll
  for (int s = 0; s < D - 1; ++s)
    if (t0 + s < nkt) XI_THIN_TILE(s, t0 + s);     // the same for every thread
#undef XI_THIN_TILE
#undef XI_THIN_ISSUE

  // ---- the four waves' sums through LDS, added in wave order.  A lane's 4 values of a tile:
  // row r of x, features 4 j .. 4 j + 3 of the tile.
#pragma unroll
  for (int t = 0; t < RT; ++t) *reinterpret_cast<f32x4*>(&red[(wave * RT + t) * 256 + lane * 4]) = acc[t];
  if constexpr (MODE == 2) {
    float t = 0.f;
#pragma unroll
    for (int i = 0; i < kThinSsLoads; ++i) t += ss_mine[i];
    t += lane_xor<8>(t);
    t += lane_xor<4>(t);
    t += lane_xor<2>(t);
    t += lane_xor<1>(t);
    if ((tid & 15) == 0) side[tid >> 4] = rsqrtf(t * fold.inv_h + fold.eps);
  }
  __syncthreads();
#pragma unroll
  for (int h = 0; h < RT; ++h) {
    const int e = tid;                       // element of feature tile h
    const int ln = e >> 2, v = e & 3;
    const int token = ln & 15, f = 16 * h + 4 * (ln >> 4) + v;      // feature within the workgroup's tile
    const int n = n0 + f;
    float a = 0.f;
#pragma unroll
    for (int wv = 0; wv < 4; ++wv) a += red[(wv * RT + h) * 256 + e];
    const bool mine = n <= n_last && token < M;
    if constexpr (MODE == 1) {
      float sq = 0.f;
      if (mine) {
        const float rr = fold.resid[(size_t)token * N + n] + a;
        fold.resid[(size_t)token * N + n] = rr;
        fold.xg[(size_t)token * N + n] = from_float<bf16>(rr * fold.g[n]);
        sq = rr * rr;
      }
      side[token * TR + f] = sq;
    } else {
      if constexpr (MODE == 2) a *= side[token];
      if (mine) y[(size_t)token * N + n] = from_float<TO>(a);
    }
  }
  if constexpr (MODE == 1) {     // a row's squares summed in the order of the features
    __syncthreads();
    if (tid < kThinRows && tid < M) {
      float t = 0.f;
      for (int i = 0; i < TR; ++i) t += side[tid * TR + i];
      fold.ss_out[(size_t)tid * gridDim.x + blockIdx.x] = t;
    }
  }
}

// Features per workgroup: the fewest workgroups that are a multiple of the 256 compute units
// with at most 32 features each.  From N alone.
static int thin_features(int N) {
  for (int waves = 1; waves <= 1024; ++waves) {
    const int rr = (N + 256 * waves - 1) / (256 * waves);
    if (rr <= kThinFeatures) return rr < 1 ? 1 : rr;
  }
  return kThinFeatures;
}

}  // namespace xi

using namespace xi;

extern "C" {

// 0 if the sizes are not taken.
int xi_linear_thin_features(int N, int K) {
  if (N < 1 || K < kThinK || K % kThinK) return 0;
  return thin_features(N);
}

// Workgroups (= parts of a row's sum of squares that xi_linear_thin_fold_out hands on).
int xi_linear_thin_parts(int N, int K) {
  const int R = xi_linear_thin_features(N, K);
  return R ? (N + R - 1) / R : 0;
}

static int thin_check(const char* what, const void* x, const void* w, int M, int N, int K) {
  XI_CHECK(M >= 1 && M <= kThinRows, "%s: M=%d must be 1..%d", what, M, kThinRows);
  XI_CHECK(N >= 1 && K >= kThinK && K % kThinK == 0, "%s: N=%d, K=%d (a multiple of %d) are not taken", what, N, K, kThinK);
  XI_CHECK(((uintptr_t)x | (uintptr_t)w) % 16 == 0, "%s: operands must be 16-byte aligned", what);
  XI_CHECK((long long)(N + thin_features(N) - 1) / thin_features(N) < (1ll << 31), "%s: too many workgroups", what);
  return 0;
}

// A tile of 16 rows of w where the workgroups own at most 16 features and K is a multiple of 512.
static int thin_tile_rows(int R, int K) { return (R <= 16 && K % 512 == 0) ? 16 : 32; }

#define XI_THIN_LAUNCH_(MODE, TO, TR, XR, yptr)                                                                      \
  do {                                                                                                          \
    static bool lds_set = false;                                                                                \
    if (!lds_set) {                                                                                             \
      hipError_t e = hipFuncSetAttribute((const void*)linear_thin_kernel<MODE, TO, TR, XR>,                         \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)thin_lds_bytes(TR));  \
      XI_CHECK(e == hipSuccess, "linear_thin: cannot get %zu bytes of LDS: %s", thin_lds_bytes(TR),             \
               hipGetErrorString(e));                                                                           \
      lds_set = true;                                                                                           \
    }                                                                                                           \
    linear_thin_kernel<MODE, TO, TR, XR><<<wgs, 256, thin_lds_bytes(TR), stream>>>(                             \
        (const bf16*)x, (const bf16*)w, (TO*)(yptr), M, N, K, R, rotate, fold);                                 \
  } while (0)
// rows of x in a tile: 4 (tiles of 16 rows of w only: their copying takes 4 rows at once), 8 or 16
#define XI_THIN_LAUNCH(MODE, TO, TR, yptr)                                    \
  do {                                                                        \
    if (M <= 4 && TR == 16) XI_THIN_LAUNCH_(MODE, TO, 16, 4, yptr);           \
    else if (M <= 8) XI_THIN_LAUNCH_(MODE, TO, TR, 8, yptr);                  \
    else XI_THIN_LAUNCH_(MODE, TO, TR, 16, yptr);                             \
  } while (0)
#define XI_THIN_TILE_ROWS(MODE, TO, yptr)                   \
  do {                                                      \
    if (thin_tile_rows(R, K) == 16) XI_THIN_LAUNCH(MODE, TO, 16, yptr); \
    else XI_THIN_LAUNCH(MODE, TO, 32, yptr);                \
  } while (0)

// y [M, N] bfloat16 (out_dtype 1) or float32 (0).
int xi_linear_thin(const void* x, const void* w, void* y, int M, int N, int K, int out_dtype, int rotate,
                   hipStream_t stream) {
  if (thin_check("linear_thin", x, w, M, N, K)) return 1;
  XI_CHECK(rotate >= 0, "linear_thin: rotate=%d", rotate);
  const int R = thin_features(N);
  const unsigned wgs = (unsigned)((N + R - 1) / R);
  const ThinFold fold{nullptr, nullptr, nullptr, nullptr, nullptr, 0, 0.f, 0.f};
  if (out_dtype == kBF16) XI_THIN_TILE_ROWS(0, bf16, y);
  else if (out_dtype == kF32) XI_THIN_TILE_ROWS(0, float, y);
  else XI_CHECK(false, "linear_thin: unknown dtype %d", out_dtype);
  XI_LAUNCH_CHECK("linear_thin");
  return 0;
}

// resid [M, N] float32 += x @ w^T; xg [M, N] = round(resid * g); ss [M, xi_linear_thin_parts(N, K)].
int xi_linear_thin_fold_out(const void* x, const void* w, int M, int N, int K, float* resid, const float* g, void* xg,
                            float* ss, int rotate, hipStream_t stream) {
  if (thin_check("linear_thin_fold_out", x, w, M, N, K)) return 1;
  XI_CHECK(resid && g && xg && ss && rotate >= 0, "linear_thin_fold_out: missing operands");
  const int R = thin_features(N);
  const unsigned wgs = (unsigned)((N + R - 1) / R);
  const ThinFold fold{resid, g, (bf16*)xg, ss, nullptr, 0, 0.f, 0.f};
  XI_THIN_TILE_ROWS(1, bf16, nullptr);
  XI_LAUNCH_CHECK("linear_thin_fold_out");
  return 0;
}

// y [M, N] = (xg @ w^T) with row t scaled by rsqrt(sum(ss[t]) / K + eps); ss [M, parts], parts <= 512.
int xi_linear_thin_fold_in(const void* x, const void* w, void* y, int M, int N, int K, int out_dtype, const float* ss,
                           int parts, float eps, int rotate, hipStream_t stream) {
  if (thin_check("linear_thin_fold_in", x, w, M, N, K)) return 1;
  XI_CHECK(ss && parts >= 1 && parts <= 16 * kThinSsLoads && rotate >= 0, "linear_thin_fold_in: %d parts (1..%d)", parts,
           16 * kThinSsLoads);
  const int R = thin_features(N);
  const unsigned wgs = (unsigned)((N + R - 1) / R);
  const ThinFold fold{nullptr, nullptr, nullptr, nullptr, ss, parts, eps, 1.f / (float)K};
  if (out_dtype == kBF16) XI_THIN_TILE_ROWS(2, bf16, y);
  else if (out_dtype == kF32) XI_THIN_TILE_ROWS(2, float, y);
  else XI_CHECK(false, "linear_thin_fold_in: unknown dtype %d", out_dtype);
  XI_LAUNCH_CHECK("linear_thin_fold_in");
  return 0;
}
#undef XI_THIN_TILE_ROWS
#undef XI_THIN_LAUNCH
#undef XI_THIN_LAUNCH_

}  // extern "C"
