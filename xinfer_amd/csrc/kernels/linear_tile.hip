// y[M, N] = x[M, K] @ w[N, K]^T in bfloat16 for many rows (prompt portions, decode steps of more
// than 128 requests) on the gfx950 matrix cores, with split K for narrow outputs.
//
// The vendor library serves these products well where the output gives it as many tiles as the
// chip has compute units; a narrow output does not (2,048 rows by 4,096 features are 128 of its
// tiles for 256 units, 256 rows 16), and its own choice of kernel does not cut K.  Here a workgroup
// of eight waves owns a tile of BM rows by BN features (128 by 256, 256 by 128, or 256 by 256) and
// one of KS slices of K, tiles x slices filling the compute units; with slices the result is
// float32 partial sums [KS, M, N] that the consumer adds in slice order (the fused add + RMSNorm,
// the q/k kernel), without them one bfloat16 rounding of the float32 sum.
//
// Tiles of 64 k reach LDS through loads that write LDS themselves (`global_load_lds_dwordx4`:
// every lane asks for one 16-byte chunk, a wave's 64 chunks land in 1 KB of consecutive LDS, no
// register holds a tile), into a ring of S stages (3, or 2 for the tile of 256 by 256: 160 KB of
// LDS); a tile is waited for with a count, not by draining the queue, and one barrier a tile orders
// the stage's reuse.  Rows of 128 bytes cannot be padded then, so the 16-byte chunks of row p are
// permuted: chunk c sits at place c ^ ((p >> 1) & 7), and the 16 lanes that read an operand together
// (16 rows, one chunk each) fall into 16 different 16-byte groups of the 64 banks (the counters
// show no bank conflict).
//
// A wave multiplies 64 features by 64 rows (128 rows in the tile of 256 by 256) as 4 x 4 (4 x 8)
// v_mfma_f32_16x16x32_bf16 tiles per 32-wide k step: A = 16 rows of w, B = 16 rows of x, so that a
// lane holds four consecutive features of one row of the result.  The operands of a tile's two
// steps live in two sets of registers, each read from LDS while the matrix cores work on the other
// set, and the loads of the tile S ahead are issued one at a time between the products: a wave that
// asks for all its loads at once waits until the load unit has taken them before it issues its
// first product (5 to 10% of the kernel's time).
//
// Measured on MI355X (random operands, the clock under load about 1.8 GHz): 2,048 rows by
// N = 4096, K = 12288 in 172 us (1.2 PFLOP/s; the library 174), K = 4096 in 68 us (the library 64);
// 4,096 x 4,096 x 4,096 in tiles of 256 by 256 108 us (1.27; the library 94); the matrix cores are
// busy 63% of the time, LDS serves the tiles' 48 to 64 KB of writes and 128 to 192 KB of reads a
// tile and is what the kernel waits for (without the barrier or without the wait for the loads it
// is no faster).  Where it is ahead of the library is the narrow output at few rows, whose tiles
// leave most of the chip idle unless K is cut: 256 rows of N = 4096, K = 12288 in 30 us against 41.
// Not kept: tiles of 32 k with two workgroups a compute unit (0.85 PFLOP/s against 0.95 at 4,096
// cubed); the tiles going memory -> registers -> LDS (0.83); four waves of twice the tile each
// (0.80); the operands of one step only in registers (the second step's reads then wait: -8%).
//
// Workgroups go round the chip's eight dies; consecutive workgroup numbers of one die are mapped
// to tiles that share rows of w, then of x, so that a die's L2 holds what its workgroups share.
// The value of an output element depends on (K, the slices) alone: never on M, on the tile shape or
// on what else is in the batch (a sum over a slice runs in ascending k, 32 at a time).
//
// Reference call site: candle matmul in /root/reference/src/models/layers/linear.rs:76-124
// (vendor BLAS).
#include "common.h"

namespace xi {

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace tile {

constexpr int kSliceK = 64;        // K is cut into slices in tiles of this many

__device__ __forceinline__ void load_lds16(const void* base, unsigned lane_off, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1" ::"v"(lane_off), "s"(base), "s"(lds_addr)
               : "memory", "m0");
}

template <int N>
__device__ __forceinline__ void wait_loads() {
  static_assert(N >= 0 && N < 64, "vmcnt has six bits");
  __builtin_amdgcn_s_waitcnt(0x0F70 | (N & 15) | ((N >> 4) << 14));
}

__device__ __forceinline__ bf16x8 lds8(const unsigned char* p) { return *reinterpret_cast<const bf16x8*>(p); }

// BM rows of x by BN rows of w a workgroup, BK = 64 k a tile; WGM x WGN waves, each (BM / WGM) by
// (BN / WGN).
template <int BM, int BN, int BK, int WGM, int WGN, int S, bool PARTIAL>
__global__ __launch_bounds__(64 * WGM * WGN, 1) void linear_tile_kernel(
    const bf16* __restrict__ x, const bf16* __restrict__ w, void* __restrict__ yv, int M, int N, int K, int tiles_m,
    int tiles_n, int slices, int k_tiles_all) {
  static_assert(BK == 64, "tiles of 64 k: rows of 128 bytes");
  constexpr int kRowBytes = BK * 2, kBK = BK;
  constexpr int CPR = BK / 8;                                // 16-byte chunks of a row
  constexpr int PS = BK == 64 ? 1 : 2;                       // rows that share a 256-byte phase differ in place: p >> PS
  constexpr int RPL = 1024 / kRowBytes;                      // rows a wave-wide load brings
  constexpr int KSTEPS = BK / 32;
  constexpr int NWV = WGM * WGN;
  constexpr int TM = BM / WGM / 16, TN = BN / WGN / 16;      // 16 x 16 tiles of a wave
  constexpr int WBYTES = BN * kRowBytes, XBYTES = BM * kRowBytes, STAGE = WBYTES + XBYTES;
  constexpr int WI = WBYTES / 1024, XI = XBYTES / 1024;      // wave-wide loads of a tile: w, then x
  static_assert((WI + XI) % NWV == 0, "every wave issues the same number of loads a tile");
  constexpr int LPW = (WI + XI) / NWV;
  static_assert(S * LPW < 64 && S >= 2, "the tiles in flight must fit the load counter");
  static_assert(BM % (16 * WGM) == 0 && BN % (16 * WGN) == 0, "whole 16 x 16 tiles a wave");
  extern __shared__ __align__(1024) unsigned char smem[];
  const unsigned lds0 = (unsigned)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int wm = wave % WGM, wn = wave / WGM;

  // ---- which tile and slice: workgroup numbers b, b + 8, b + 16, .. run on one die; they get
  // consecutive places in the order (slice, tile of features, tile of rows)
  const int total = tiles_m * tiles_n * slices;
  int place = blockIdx.x;
  if (total % 8 == 0) place = (blockIdx.x & 7) * (total >> 3) + (blockIdx.x >> 3);
  const int per_slice = tiles_m * tiles_n;
  const int slice = place / per_slice;
  const int in_slice = place - slice * per_slice;
  const int tn_i = in_slice / tiles_m, tm_i = in_slice - tn_i * tiles_m;
  const int m0 = tm_i * BM, n0 = tn_i * BN;
  // slice s of the K / 64 tiles: [s * tiles / slices, (s + 1) * tiles / slices), one tile at least
  const int kt_begin = (int)((long long)slice * k_tiles_all / slices);
  const int k_tiles = (int)((long long)(slice + 1) * k_tiles_all / slices) - kt_begin;
  const size_t k0 = (size_t)kt_begin * BK;

  // ---- what this lane brings of every tile: per load of its wave the byte offset of its chunk from
  // the tile's first element of w (or x); rows past the end are read from the last row (nobody
  // stores what they make)
  unsigned ld_off[LPW];
#pragma unroll
  for (int t = 0; t < LPW; ++t) {
    const int ii = wave + NWV * t;
    const bool is_w = ii < WI;
    const int p = RPL * (is_w ? ii : ii - WI) + lane / CPR;      // row within the operand's tile
    const int ch = (lane % CPR) ^ ((p >> PS) & (CPR - 1));       // the chunk that belongs at this lane's place
    int row = (is_w ? n0 : m0) + p;
    const int last = (is_w ? N : M) - 1;
    row = row > last ? last : row;
    ld_off[t] = (unsigned)(((size_t)(row - (is_w ? n0 : m0)) * K) * 2 + ch * 16);
  }
  const bf16* wbase = w + (size_t)n0 * K + k0;
  const bf16* xbase = x + (size_t)m0 * K + k0;

  // the t-th of this wave's loads of tile kt, into stage st
  auto fetch_one = [&](int kt, int st, int t) {
    const int ii = wave + NWV * t;
    // (which operand a wave's t-th load takes is the same in all its lanes: made a scalar by hand)
    const unsigned long long a = (unsigned long long)(uintptr_t)((ii < WI ? wbase : xbase) + (size_t)kt * kBK);
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    load_lds16(reinterpret_cast<const void*>((uintptr_t)(((unsigned long long)hi << 32) | lo)), ld_off[t],
               __builtin_amdgcn_readfirstlane(lds0 + (unsigned)st * STAGE + (unsigned)ii * 1024u));
  };
  auto fetch = [&](int kt, int st) {
#pragma unroll
    for (int t = 0; t < LPW; ++t) fetch_one(kt, st, t);
  };

  // where this lane reads its operands within a stage: row r of a 16-row tile, chunk 4 ks + j at
  // its permuted place (16 rows further on the permutation is the same)
  unsigned rd[KSTEPS];
#pragma unroll
  for (int ks = 0; ks < KSTEPS; ++ks) rd[ks] = (unsigned)(r * kRowBytes + 16 * ((4 * ks + j) ^ ((r >> PS) & (CPR - 1))));
  const unsigned w_rd = (unsigned)(wn * TN * 16) * kRowBytes;
  const unsigned x_rd = WBYTES + (unsigned)(wm * TM * 16) * kRowBytes;

  f32x4 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

  auto read = [&](const unsigned char* T, int ks, bf16x8 (&wa)[TN], bf16x8 (&xb)[TM]) {
#pragma unroll
    for (int a = 0; a < TN; ++a) wa[a] = lds8(T + w_rd + rd[ks] + a * 16 * kRowBytes);
#pragma unroll
    for (int b = 0; b < TM; ++b) xb[b] = lds8(T + x_rd + rd[ks] + b * 16 * kRowBytes);
  };
  auto multiply = [&](const bf16x8 (&wa)[TN], const bf16x8 (&xb)[TM]) {
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
      for (int b = 0; b < TM; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa[a], xb[b], acc[a][b], 0, 0, 0);
  };

  // The walk, one barrier a tile.  A tile's two 32-wide steps have their operands in two sets of
  // registers; each set is read from LDS while the matrix cores work on the other: the second
  // step's before the first step's products are issued, the next tile's first step's (behind the
  // barrier that says the tile has landed) before the second step's products.  Tiles past the
  // slice's last are asked for all the same (from the last one's place) and read too, so that the
  // number of loads in flight and the code do not depend on where the walk is.
  static_assert(KSTEPS == 2, "two sets of operand registers, one a step");
#pragma unroll
  for (int p = 0; p < S; ++p) fetch(p < k_tiles ? p : k_tiles - 1, p);
  bf16x8 wa0[TN], xb0[TM], wa1[TN], xb1[TM];
  wait_loads<(S - 1) * LPW>();       // this wave's loads of the first tile have landed
  __syncthreads();                   // everybody's have
  read(smem, 0, wa0, xb0);
  int st = 0;
  for (int kt = 0; kt < k_tiles; ++kt) {
    const unsigned char* T = smem + (size_t)st * STAGE;
    read(T, 1, wa1, xb1);
    __builtin_amdgcn_sched_barrier(0);
    multiply(wa0, xb0);
    __builtin_amdgcn_sched_barrier(0);
    wait_loads<(S - 2) * LPW>();     // this wave's loads of the next tile have landed, and its reads of this one
    __builtin_amdgcn_s_waitcnt(0xC07F);   // (lgkmcnt(0): the operands above are in registers)
    __syncthreads();                 // everybody's: the next tile is whole, and this tile's stage is free
    const int filled = st;
    const int nxt = kt + S < k_tiles ? kt + S : k_tiles - 1;
    st = st + 1 == S ? 0 : st + 1;
    read(smem + (size_t)st * STAGE, 0, wa0, xb0);
    __builtin_amdgcn_sched_barrier(0);
    // the second step's products with the loads of the tile S ahead between them: a wave that asks
    // for all its loads at once waits until the load unit has taken them (it takes a compute unit's
    // 48 to 64 KB a tile at about 55 bytes a clock) before it issues its first product
    {
      constexpr int PER = (TN * TM) / LPW;       // products between two loads
#pragma unroll
      for (int a = 0; a < TN; ++a)
#pragma unroll
        for (int b = 0; b < TM; ++b) {
          const int idx = a * TM + b;
          if (idx % PER == 0 && idx / PER < LPW) {
            __builtin_amdgcn_sched_barrier(0);
            fetch_one(nxt, filled, idx / PER);
          }
          acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wa1[a], xb1[b], acc[a][b], 0, 0, 0);
        }
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  wait_loads<0>();     // the tiles asked for past the end are still on their way into LDS

  // ---- a lane holds features n .. n + 3 of row m of every 16 x 16 tile
  const int mw = m0 + wm * TM * 16 + r, nw = n0 + wn * TN * 16 + 4 * j;
#pragma unroll
  for (int b = 0; b < TM; ++b) {
    const int m = mw + 16 * b;
    if (m >= M) continue;
#pragma unroll
    for (int a = 0; a < TN; ++a) {
      const int n = nw + 16 * a;
      if (n >= N) continue;          // (N is a multiple of 4)
      const f32x4 v = acc[a][b];
      if (PARTIAL) {
        float* y = reinterpret_cast<float*>(yv) + ((size_t)slice * M + m) * N + n;
        *reinterpret_cast<f32x4*>(y) = v;
      } else {
        bf16* y = reinterpret_cast<bf16*>(yv) + (size_t)m * N + n;
        typedef __attribute__((ext_vector_type(4))) __bf16 bf16x4;
        bf16x4 o;
        o[0] = (__bf16)v[0];
        o[1] = (__bf16)v[1];
        o[2] = (__bf16)v[2];
        o[3] = (__bf16)v[3];
        *reinterpret_cast<bf16x4*>(y) = o;
      }
    }
  }
}


}  // namespace tile
}  // namespace xi

using namespace xi;

extern "C" {

// Whether the tiled product takes a shape: K in whole tiles of 64, a tile a slice at least, N in fours.
int xi_linear_tile_takes(int M, int N, int K, int slices) {
  return M > 0 && N > 0 && N % 4 == 0 && slices >= 1 && K > 0 && K % tile::kSliceK == 0 && K / tile::kSliceK >= slices;
}

// x [M, K], w [N, K] bfloat16.  slices == 1 and partial == 0: y bfloat16 [M, N].  Otherwise y is
// float32 [slices, M, N], the sums over the slices of K: slice s takes the tiles of 64 k from
// s * (K / 64) / slices up to (s + 1) * (K / 64) / slices (whole numbers: the slices differ by a tile
// at most).  shape 0: tiles of 128 rows by 256
// features; 1: 256 rows by 128 features; 2: 256 by 256.
int xi_linear_tile(const void* x, const void* w, void* y, int M, int N, int K, int slices, int partial, int shape,
                   hipStream_t stream) {
  XI_CHECK(xi_linear_tile_takes(M, N, K, slices), "linear_tile: M=%d N=%d K=%d in %d slices is not taken (K in tiles of "
           "64, a tile a slice at least, N a multiple of 4)", M, N, K, slices);
  XI_CHECK(partial || slices == 1, "linear_tile: %d slices need the float32 partial sums", slices);
  XI_CHECK(shape >= 0 && shape <= 2, "linear_tile: unknown tile shape %d", shape);
  XI_CHECK((size_t)K * 2 * 256 < ((size_t)1 << 32), "linear_tile: K=%d is too long for 32-bit offsets within a tile", K);
  const int bm = shape == 0 ? 128 : 256, bn = shape == 1 ? 128 : 256;
  const int tiles_m = (M + bm - 1) / bm, tiles_n = (N + bn - 1) / bn;
  const long long total = (long long)tiles_m * tiles_n * slices;
  XI_CHECK(total <= 0x7fffffffLL, "linear_tile: too many workgroups");
#define XI_TILE(BM, BN, BK, WGM, WGN, S, PARTIAL)                                                                 \
  do {                                                                                                            \
    auto kern = tile::linear_tile_kernel<BM, BN, BK, WGM, WGN, S, PARTIAL>;                                        \
    const size_t lds = (size_t)(S) * (BM + BN) * BK * 2;                                                          \
    hipError_t e = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);  \
    XI_CHECK(e == hipSuccess, "linear_tile: cannot get %zu bytes of LDS: %s", lds, hipGetErrorString(e));         \
    kern<<<(unsigned)total, 64 * WGM * WGN, lds, stream>>>((const bf16*)x, (const bf16*)w, y, M, N, K, tiles_m,   \
                                                           tiles_n, slices, K / BK);                   \
  } while (0)
  if (shape == 0) {
    if (partial) XI_TILE(128, 256, 64, 2, 4, 3, true);
    else XI_TILE(128, 256, 64, 2, 4, 3, false);
  } else if (shape == 1) {
    if (partial) XI_TILE(256, 128, 64, 4, 2, 3, true);
    else XI_TILE(256, 128, 64, 4, 2, 3, false);
  } else {
    if (partial) XI_TILE(256, 256, 64, 2, 4, 2, true);
    else XI_TILE(256, 256, 64, 2, 4, 2, false);
  }
#undef XI_TILE
  XI_LAUNCH_CHECK("linear_tile");
  return 0;
}

}  // extern "C"
