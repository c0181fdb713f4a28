// y[M,N] = x[M,K] @ w[N,K]^T in bfloat16 for few rows (decode batches): bound by the one
// pass over w, so the kernel is a streaming read of w through the matrix cores.
//
// One workgroup owns 16*RT rows of w (output features) over all of K; its NW waves take
// consecutive K ranges and merge through LDS in wave order, so an output element's value
// depends on (K, NW) alone, never on M or on what else is in the batch.  Per 32-wide k
// step a wave issues v_mfma_f32_16x16x32_bf16 with A = 16 rows of w (lane l: row l%16,
// k group l/16, one 16-byte load) and B = x^T (lane l: token l%16, same k group), for
// MT tiles of 16 tokens.  x is small (M <= 64 rows) and is read from L2 by every wave.
//
// GATED: w is [2N, K] = [gate; up]; the workgroup computes rows n (gate) and N + n (up)
// and stores silu(gate) * up, float32 math and one rounding, so the packed [M, 2N]
// intermediate of the feed-forward never goes to memory.
//
// Reference call sites: candle matmul in /root/reference/src/models/layers/linear.rs:76-124
// (vendor BLAS); fused gate/up + silu_and_mul in /root/reference/src/models/layers/mlp.rs:613-633.
#include "common.h"

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

template <int MT, int RT, int NW, int U, bool GATED, typename TO>
__global__ __launch_bounds__(NW * 64) void linear_skinny_kernel(const bf16* __restrict__ x,
                                                                const bf16* __restrict__ w,
                                                                TO* __restrict__ y, int M, int N, int K) {
  static_assert(!GATED || RT == 2, "the gated form pairs one gate tile with one up tile");
  __shared__ float red[NW * RT * MT * 256];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, j = lane >> 4;
  const int n0 = blockIdx.x * (GATED ? 16 : 16 * RT);

  // rows of w and x this lane loads; rows past the end are clamped (their results are dropped)
  const bf16* wp[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) {
    int row = GATED ? (t == 0 ? n0 + r : N + n0 + r) : n0 + 16 * t + r;
    const int last = GATED ? (t == 0 ? N - 1 : 2 * N - 1) : N - 1;
    if (row > last) row = last;
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
  const int per = (steps + NW - 1) / NW;
  const int s0 = wave * per;
  const int s1 = min(steps, s0 + per);
  const int s_fast = min(s1, steps_full);
  int s = s0;
  for (; s + U <= s_fast; s += U) {
    bf16x8 a[RT][U], b[MT][U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int t = 0; t < RT; ++t) a[t][u] = ldg8(wp[t] + 32 * (s + u));
#pragma unroll
      for (int m = 0; m < MT; ++m) b[m][u] = ldg8(xp[m] + 32 * (s + u));
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
#pragma unroll
      for (int t = 0; t < RT; ++t)
#pragma unroll
        for (int m = 0; m < MT; ++m)
          acc[t][m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[t][u], b[m][u], acc[t][m], 0, 0, 0);
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

  // lane holds token r, features 4j..4j+3 of each tile
#pragma unroll
  for (int t = 0; t < RT; ++t)
#pragma unroll
    for (int m = 0; m < MT; ++m)
      *reinterpret_cast<f32x4*>(&red[((wave * RT + t) * MT + m) * 256 + r * 16 + 4 * j]) = acc[t][m];
  __syncthreads();

  if (GATED) {
    for (int idx = threadIdx.x; idx < MT * 256; idx += NW * 64) {
      const int m = idx >> 8, tok = (idx >> 4) & 15, f = idx & 15;
      float g = 0.f, u = 0.f;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) {
        g += red[((wv * RT + 0) * MT + m) * 256 + tok * 16 + f];
        u += red[((wv * RT + 1) * MT + m) * 256 + tok * 16 + f];
      }
      const int token = 16 * m + tok, n = n0 + f;
      if (token < M && n < N) y[(size_t)token * N + n] = from_float<TO>(g / (1.f + __expf(-g)) * u);
    }
  } else {
    for (int idx = threadIdx.x; idx < RT * MT * 256; idx += NW * 64) {
      const int t = idx / (MT * 256), rem = idx - t * (MT * 256);
      const int m = rem >> 8, tok = (rem >> 4) & 15, f = rem & 15;
      float sum = 0.f;
#pragma unroll
      for (int wv = 0; wv < NW; ++wv) sum += red[((wv * RT + t) * MT + m) * 256 + tok * 16 + f];
      const int token = 16 * m + tok, n = n0 + 16 * t + f;
      if (token < M && n < N) y[(size_t)token * N + n] = from_float<TO>(sum);
    }
  }
}

template <int MT, int RT, int NW, int U, bool GATED, typename TO>
static void launch_skinny(const void* x, const void* w, void* y, int M, int N, int K, hipStream_t stream) {
  const int rows_per_wg = GATED ? 16 : 16 * RT;
  const unsigned grid = (unsigned)((N + rows_per_wg - 1) / rows_per_wg);
  linear_skinny_kernel<MT, RT, NW, U, GATED, TO><<<grid, NW * 64, 0, stream>>>(
      (const bf16*)x, (const bf16*)w, (TO*)y, M, N, K);
}

}  // namespace xi

using namespace xi;

extern "C" {

// Most rows of x the skinny kernels take.
int xi_linear_skinny_max_rows() { return 64; }

// x [M, K] bf16, w [N, K] bf16 -> y [M, N] in out_dtype (bf16 or float32).
// gated != 0: w is [2N, K] and y [M, N] = silu(x @ w[:N]^T) * (x @ w[N:]^T).
// variant: 0 = chosen from the sizes; other values select a tile shape (for measurements).
int xi_linear_skinny(const void* x, const void* w, void* y, int M, int N, int K, int out_dtype, int gated,
                     int variant, hipStream_t stream) {
  XI_CHECK(M >= 0 && N > 0 && K > 0, "linear_skinny: bad sizes M=%d N=%d K=%d", M, N, K);
  XI_CHECK(M <= 64, "linear_skinny: %d rows exceed 64 (use the library product)", M);
  XI_CHECK(K % 8 == 0, "linear_skinny: K=%d must be a multiple of 8", K);
  XI_CHECK(out_dtype == kBF16 || out_dtype == kF32, "linear_skinny: unknown output dtype %d", out_dtype);
  if (M == 0) return 0;
  const int mt = (M + 15) / 16;
  const int tiles = (N + 15) / 16;  // 16-row tiles of the output
  // Wide outputs keep two row tiles per workgroup (x operands are reused); narrow ones one
  // tile and sixteen waves so that every compute unit still has work.  The number of waves
  // fixes the order of the float32 sums, so it is chosen from N alone and a row's result
  // does not depend on how many rows came with it (the gated form with more than 32 rows
  // is the exception: sixteen waves of two tiles do not fit in LDS there).
  int rt = (variant == 1) ? 1 : (variant == 2) ? 2 : (tiles >= 2048 ? 2 : 1);
  if (gated) rt = 2;
  int nw = (variant == 3) ? 16 : (variant == 4) ? 8 : ((gated ? tiles : tiles / rt) < 512 ? 16 : 8);
  if (nw == 16 && rt * mt > 4) {
    if (rt == 2 && !gated && variant != 2) rt = 1;
    else nw = 8;
  }
#define XI_SK(MT, RT, NW, U, G, TO) launch_skinny<MT, RT, NW, U, G, TO>(x, w, y, M, N, K, stream)
#define XI_SK_TO(MT, RT, NW, U, G)                         \
  do {                                                     \
    if (out_dtype == kBF16) XI_SK(MT, RT, NW, U, G, bf16); \
    else XI_SK(MT, RT, NW, U, G, float);                   \
  } while (0)
#define XI_SK_MT(RT, NW, G)                                   \
  do {                                                        \
    if (mt == 1) XI_SK_TO(1, RT, NW, (RT == 1 ? 8 : 4), G);   \
    else if (mt == 2) XI_SK_TO(2, RT, NW, 4, G);              \
    else if (mt == 3) XI_SK_TO(3, RT, NW, (RT == 1 ? 4 : 2), G); \
    else XI_SK_TO(4, RT, NW, (RT == 1 ? 4 : 2), G);           \
  } while (0)
  if (gated) {
    if (nw == 16) {
      if (mt == 1) XI_SK_TO(1, 2, 16, 4, true);
      else XI_SK_TO(2, 2, 16, 4, true);
    } else {
      XI_SK_MT(2, 8, true);
    }
  } else if (rt == 2) {
    if (nw == 16) {
      if (mt == 1) XI_SK_TO(1, 2, 16, 4, false);
      else XI_SK_TO(2, 2, 16, 4, false);
    } else {
      XI_SK_MT(2, 8, false);
    }
  } else {
    if (nw == 16) XI_SK_MT(1, 16, false);
    else XI_SK_MT(1, 8, false);
  }
#undef XI_SK_MT
#undef XI_SK_TO
#undef XI_SK
  XI_LAUNCH_CHECK("linear_skinny");
  return 0;
}

}  // extern "C"
