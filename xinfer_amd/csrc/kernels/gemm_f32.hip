// y[M,N] = x[M,K] @ w[N,K]^T with float32 accumulation in ascending k by one fma chain
// per output element: the value of an element does not depend on M, on the tile it
// falls in, or on what else is in the batch.  This is the matrix product of the true
// 32-bit path (no reduced-precision matrix mode); it also accepts bfloat16 operands.
// Reference call site: candle matmul, /root/reference/src/models/layers/linear.rs:76-124.
#include "common.h"

namespace xi {

constexpr int BM = 64, BN = 64, BK = 16, TM = 4, TN = 4;

template <typename TI, typename TO, bool ADD>
__global__ __launch_bounds__(256) void gemm_tn_kernel(const TI* __restrict__ x,
                                                      const TI* __restrict__ w,
                                                      TO* __restrict__ y, int M, int N, int K) {
  __shared__ float xs[BK][BM + 4];
  __shared__ float ws[BK][BN + 4];
  const int tid = threadIdx.x;
  const int m0 = blockIdx.y * BM;
  const int n0 = blockIdx.x * BN;
  const int tx = tid % 16;  // n direction
  const int ty = tid / 16;  // m direction
  float acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) acc[i][j] = 0.f;

  const int lr = tid / 4;        // 0..63: row of the tile this thread loads
  const int lk = (tid % 4) * 4;  // 0,4,8,12: first k of the four it loads
  for (int k0 = 0; k0 < K; k0 += BK) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int k = k0 + lk + q;
      const int m = m0 + lr;
      const int n = n0 + lr;
      xs[lk + q][lr] = (m < M && k < K) ? to_float(x[(size_t)m * K + k]) : 0.f;
      ws[lk + q][lr] = (n < N && k < K) ? to_float(w[(size_t)n * K + k]) : 0.f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < BK; ++kk) {
      float a[TM], b[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) a[i] = xs[kk][ty * TM + i];
#pragma unroll
      for (int j = 0; j < TN; ++j) b[j] = ws[kk][tx * TN + j];
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = fmaf(a[i], b[j], acc[i][j]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < TM; ++i) {
    const int m = m0 + ty * TM + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < TN; ++j) {
      const int n = n0 + tx * TN + j;
      if (n >= N) continue;
      const size_t o = (size_t)m * N + n;
      if (ADD)
        y[o] = from_float<TO>(to_float(y[o]) + acc[i][j]);
      else
        y[o] = from_float<TO>(acc[i][j]);
    }
  }
}

}  // namespace xi

using namespace xi;

extern "C" int xi_gemm_tn(const void* x, const void* w, void* y, int M, int N, int K, int in_dtype,
                          int out_dtype, int accumulate, hipStream_t stream) {
  XI_CHECK(M >= 0 && N > 0 && K > 0, "gemm: bad sizes M=%d N=%d K=%d", M, N, K);
  if (M == 0) return 0;
  dim3 grid((N + BN - 1) / BN, (M + BM - 1) / BM);
  XI_CHECK(grid.y <= 65535u, "gemm: M=%d is too large for one launch", M);
#define XI_GEMM(TI, TO)                                                                         \
  do {                                                                                          \
    if (accumulate)                                                                             \
      gemm_tn_kernel<TI, TO, true><<<grid, 256, 0, stream>>>((const TI*)x, (const TI*)w, (TO*)y, M, N, K); \
    else                                                                                        \
      gemm_tn_kernel<TI, TO, false><<<grid, 256, 0, stream>>>((const TI*)x, (const TI*)w, (TO*)y, M, N, K); \
  } while (0)
  if (in_dtype == kF32 && out_dtype == kF32) XI_GEMM(float, float);
  else if (in_dtype == kBF16 && out_dtype == kBF16) XI_GEMM(bf16, bf16);
  else if (in_dtype == kBF16 && out_dtype == kF32) XI_GEMM(bf16, float);
  else XI_CHECK(false, "gemm: unsupported dtypes in=%d out=%d", in_dtype, out_dtype);
#undef XI_GEMM
  XI_LAUNCH_CHECK("gemm");
  return 0;
}
