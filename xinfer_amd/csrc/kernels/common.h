// Shared helpers of the gfx950 kernels: element types, wave64 reductions, error reporting.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_bf16.h>
#include <stdint.h>

namespace xi {

constexpr int kWave = 64;  // CDNA wavefront width

enum DType : int { kF32 = 0, kBF16 = 1 };

using bf16 = __hip_bfloat16;

// ---- element load/store in float ------------------------------------------------
__device__ __forceinline__ float to_float(float v) { return v; }
__device__ __forceinline__ float to_float(bf16 v) { return __bfloat162float(v); }

template <typename T> __device__ __forceinline__ T from_float(float v);
template <> __device__ __forceinline__ float from_float<float>(float v) { return v; }
template <> __device__ __forceinline__ bf16 from_float<bf16>(float v) { return __float2bfloat16(v); }

// ---- wave64 reductions in a fixed order ----------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = kWave / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, kWave));
  return v;
}

// Sum over a whole workgroup of `NW` waves; every thread gets the result.  `scratch`
// holds NW floats of LDS.  The order of additions is fixed by the thread layout alone.
template <int NW>
__device__ __forceinline__ float block_sum(float v, float* scratch) {
  v = wave_sum(v);
  const int wave = threadIdx.x / kWave;
  __syncthreads();
  if ((threadIdx.x & (kWave - 1)) == 0) scratch[wave] = v;
  __syncthreads();
  float total = 0.f;
#pragma unroll
  for (int i = 0; i < NW; ++i) total += scratch[i];
  return total;
}

// ---- error reporting to the host caller -------------------------------------------
void set_error(const char* fmt, ...);

}  // namespace xi

#define XI_CHECK(cond, ...)            \
  do {                                 \
    if (!(cond)) {                     \
      xi::set_error(__VA_ARGS__);      \
      return 1;                        \
    }                                  \
  } while (0)

#define XI_LAUNCH_CHECK(name)                                                \
  do {                                                                       \
    hipError_t e_ = hipGetLastError();                                       \
    if (e_ != hipSuccess) {                                                  \
      xi::set_error("%s: launch failed: %s", name, hipGetErrorString(e_));   \
      return 2;                                                              \
    }                                                                        \
  } while (0)
