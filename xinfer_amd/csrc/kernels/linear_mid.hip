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
// Reference call site: candle matmul in /root/reference/src/models/layers/linear.rs:76-124
// (vendor BLAS).
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

constexpr int kMidRows = 128;          // rows of x a workgroup takes: all of them
constexpr int kMidFeatures = 128;      // output features of a workgroup
constexpr int kMidK = 64;              // k per tile
constexpr int kMidLdsRow = kMidK + 8;  // elements of a row in LDS
constexpr int kMidDepth = 2;           // tiles whose loads are in flight (the default; measured: more gain nothing)
constexpr int kMidTile = 128 * kMidLdsRow;   // elements of one operand's tile in LDS
constexpr size_t kMidLdsBytes = 2 * 2 * (size_t)kMidTile * sizeof(bf16);

// D: tiles whose loads are in flight.  HALF: at most 64 rows of x; the four waves then take a
// quarter of the features each (32 features by 64 rows) instead of a quarter of the tile.
template <int D, bool HALF>
__global__ __launch_bounds__(256, 1) void linear_mid_kernel(const bf16* __restrict__ x,
                                                            const bf16* __restrict__ w, float* __restrict__ y,
                                                            int M, int N, int K, int ks, size_t slice_stride) {
  extern __shared__ __align__(16) unsigned char mid_smem[];
  bf16* lds = reinterpret_cast<bf16*>(mid_smem);   // [buffer][w tile | x tile][128][kMidLdsRow]
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  constexpr int TI = HALF ? 2 : 4;                    // 16-feature tiles of a wave
  const int wf = HALF ? wave : (wave & 1);            // the wave's features start at 16 * TI * wf,
  const int wt = HALF ? 0 : (wave >> 1);              // its rows at 64 * wt
  const int slice = blockIdx.x % ks, tile = blockIdx.x / ks;
  const int n0 = tile * kMidFeatures;
  // the k tiles of this slice: K / 64 tiles dealt out as evenly as they go
  const int kt_total = K / kMidK;
  const int base = kt_total / ks, rem = kt_total % ks;
  const int kt0 = slice * base + (slice < rem ? slice : rem);
  const int nkt = base + (slice < rem ? 1 : 0);

  // ---- copying: a tile is 128 rows of 8 16-byte chunks; thread t moves chunk t % 8 of rows
  // t / 8 + 32 i.  Rows of w past N read row N - 1 again and rows of x past M row M - 1 (the
  // same address many times in one instruction costs one access); their results are dropped.
  // No load is conditional, so the counter of loads in flight is exact and only the tile that
  // is needed is waited for.
  const int srow = tid >> 3, skc = tid & 7;
  const bf16* wsrc[4];
  const bf16* xsrc[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = srow + 32 * i;
    int n = n0 + row;
    n = n < N ? n : N - 1;
    wsrc[i] = w + (size_t)n * K + (size_t)kt0 * kMidK + 8 * skc;
    xsrc[i] = x + (size_t)(row < M ? row : M - 1) * K + (size_t)kt0 * kMidK + 8 * skc;
  }
  const int sdst = srow * kMidLdsRow + 8 * skc;
  bf16x8 wr[D][4], xr[D][4];

  // a wave whose half of the rows lies past M has nothing to multiply
  const bool active = __builtin_amdgcn_readfirstlane(64 * wt < M ? 1 : 0) != 0;
  f32x4 acc[TI][4];
#pragma unroll
  for (int ti = 0; ti < TI; ++ti)
#pragma unroll
    for (int tj = 0; tj < 4; ++tj) acc[ti][tj] = f32x4{0.f, 0.f, 0.f, 0.f};

#define XI_MID_ISSUE(slot, t)                                                         \
  do {                                                                                \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                   \
      wr[slot][i] = *reinterpret_cast<const bf16x8*>(wsrc[i] + (size_t)(t) * kMidK);  \
      xr[slot][i] = *reinterpret_cast<const bf16x8*>(xsrc[i] + (size_t)(t) * kMidK);  \
    }                                                                                 \
  } while (0)

  // Every copy is issued whether or not its tile exists (past the slice's end the last tile is
  // read again, from cache, and dropped): with a fixed number of loads between a tile's loads
  // and its use, the wait before the use leaves exactly the younger tiles in flight.
  const int last = nkt - 1;
#pragma unroll
  for (int s = 0; s < D; ++s) XI_MID_ISSUE(s, s < last ? s : last);

  // One tile: registers of slot s to LDS, the slot loaded again kMidDepth tiles ahead, barrier,
  // products.  One barrier a tile is enough: whoever writes this buffer again, two tiles on, has
  // passed the next tile's barrier, which every thread reaches only after these products.
  int buf = 0;
#define XI_MID_TILE(s, t)                                                                                 \
  do {                                                                                                    \
    bf16* Ws = lds + buf * (2 * kMidTile);                                                                \
    bf16* Xs = Ws + kMidTile;                                                                             \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                                       \
      *reinterpret_cast<bf16x8*>(Ws + sdst + 32 * i * kMidLdsRow) = wr[s][i];                             \
      *reinterpret_cast<bf16x8*>(Xs + sdst + 32 * i * kMidLdsRow) = xr[s][i];                             \
    }                                                                                                     \
    XI_MID_ISSUE(s, (t) + D < last ? (t) + D : last);                                                     \
    __syncthreads();                                                                                      \
    if (active) {                                                                                         \
      _Pragma("unroll") for (int kk = 0; kk < kMidK / 32; ++kk) {                                         \
        bf16x8 a[TI], b[4];                                                                               \
        _Pragma("unroll") for (int ti = 0; ti < TI; ++ti) a[ti] = *reinterpret_cast<const bf16x8*>(       \
            Ws + (16 * TI * wf + 16 * ti + r) * kMidLdsRow + 32 * kk + 8 * j);                            \
        _Pragma("unroll") for (int tj = 0; tj < 4; ++tj) b[tj] = *reinterpret_cast<const bf16x8*>(        \
            Xs + (64 * wt + 16 * tj + r) * kMidLdsRow + 32 * kk + 8 * j);                                 \
        _Pragma("unroll") for (int ti = 0; ti < TI; ++ti)                                                 \
          _Pragma("unroll") for (int tj = 0; tj < 4; ++tj)                                                \
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

  // a lane's 4 values of a tile: row 16 tj + r of x, features 4 j .. 4 j + 3
  float* ys = y + (size_t)slice * slice_stride;
  const bool vec = (N & 3) == 0;
#pragma unroll
  for (int tj = 0; tj < 4; ++tj) {
    const int token = 64 * wt + 16 * tj + r;
    if (token >= M) continue;
#pragma unroll
    for (int ti = 0; ti < TI; ++ti) {
      const int f = n0 + 16 * TI * wf + 16 * ti + 4 * j;
      float* dst = ys + (size_t)token * N + f;
      if (vec && f + 3 < N) {
        *reinterpret_cast<f32x4*>(dst) = acc[ti][tj];
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (f + i < N) dst[i] = acc[ti][tj][i];
      }
    }
  }
}

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

}  // namespace xi

using namespace xi;

extern "C" {

int xi_linear_mid_max_rows() { return 2 * kMidRows; }

// 0 if the sizes are not taken (the caller then uses another product).
int xi_linear_mid_slices(int N, int K) {
  if (N < 1 || K < kMidK || K % kMidK) return 0;
  return mid_slices(N, K);
}

// y: float32 [slices, M, N] with slices = xi_linear_mid_slices(N, K).  Up to 256 rows: blocks of
// 128 rows are launched one after the other (the second pass over w comes in part from the
// last level cache).  depth: tiles of loads in flight, 0 = the default (the result does not
// depend on it).
int xi_linear_mid(const void* x, const void* w, float* y, int M, int N, int K, int depth, hipStream_t stream) {
  XI_CHECK(M >= 1 && M <= 2 * kMidRows, "linear_mid: M=%d must be 1..%d", M, 2 * kMidRows);
  XI_CHECK(N >= 1 && K >= kMidK && K % kMidK == 0, "linear_mid: N=%d, K=%d (a multiple of %d) are not taken", N, K, kMidK);
  XI_CHECK(((uintptr_t)x | (uintptr_t)w | (uintptr_t)y) % 16 == 0, "linear_mid: operands must be 16-byte aligned");
  const int ks = mid_slices(N, K);
  const long long tiles = (N + kMidFeatures - 1) / kMidFeatures;
  XI_CHECK(ks >= 1 && ks <= K / kMidK, "linear_mid: %d slices for K=%d", ks, K);
  XI_CHECK(tiles * ks < (1ll << 31), "linear_mid: too many workgroups");
  if (depth == 0) depth = kMidDepth;
#define XI_MID(D, HALF)                                                                                       \
  do {                                                                                                        \
    static bool lds_set = false;                                                                              \
    if (!lds_set) {                                                                                           \
      hipError_t e = hipFuncSetAttribute((const void*)linear_mid_kernel<D, HALF>,                             \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)kMidLdsBytes);      \
      XI_CHECK(e == hipSuccess, "linear_mid: cannot get %zu bytes of LDS: %s", kMidLdsBytes,                  \
               hipGetErrorString(e));                                                                         \
      lds_set = true;                                                                                         \
    }                                                                                                         \
    linear_mid_kernel<D, HALF><<<(unsigned)(tiles * ks), 256, kMidLdsBytes, stream>>>(                        \
        (const bf16*)x + (size_t)row0 * K, (const bf16*)w, y + (size_t)row0 * N, rows, N, K, ks,              \
        (size_t)M * N);                                                                                       \
  } while (0)
#define XI_MID_D(D)                                        \
  do {                                                     \
    for (int row0 = 0; row0 < M; row0 += kMidRows) {       \
      const int rows = M - row0 < kMidRows ? M - row0 : kMidRows; \
      if (rows <= 64) XI_MID(D, true);                     \
      else XI_MID(D, false);                               \
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

}  // extern "C"
