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

// ---- the value of lane (l ^ OFF), OFF a power of two, without the LDS pipe --------------------
// What __shfl_xor gives (it compiles to ds_bpermute_b32, a trip through the LDS crossbar), from
// gfx950's lane-swap instructions (16, 32) and data-parallel moves within a row of 16 lanes.
template <int CTRL, int BANKS>
__device__ __forceinline__ unsigned dpp_move(unsigned old, unsigned v) {
  return (unsigned)__builtin_amdgcn_update_dpp((int)old, (int)v, CTRL, 0xF, BANKS, false);
}
template <int OFF>
__device__ __forceinline__ unsigned lane_xor_bits(unsigned v) {
  static_assert(OFF == 1 || OFF == 2 || OFF == 4 || OFF == 8 || OFF == 16 || OFF == 32, "a power of two below 64");
  if constexpr (OFF == 32) {          // the two halves of the wave change places
    const auto r = __builtin_amdgcn_permlane32_swap(v, v, false, false);
    return (threadIdx.x & 32) ? r[0] : r[1];
  } else if constexpr (OFF == 16) {   // odd and even rows change places
    const auto r = __builtin_amdgcn_permlane16_swap(v, v, false, false);
    return (threadIdx.x & 16) ? r[0] : r[1];
  } else if constexpr (OFF == 8) {    // row_ror:8
    return dpp_move<0x128, 0xF>(v, v);
  } else if constexpr (OFF == 4) {    // lanes 0-3 and 8-11 of a row from 4 above (row_shl:4), the others from 4 below (row_shr:4)
    const unsigned up = dpp_move<0x104, 0x5>(v, v);
    return dpp_move<0x114, 0xA>(up, v);
  } else if constexpr (OFF == 2) {    // quad_perm [2, 3, 0, 1]
    return dpp_move<0x4E, 0xF>(v, v);
  } else {                            // quad_perm [1, 0, 3, 2]
    return dpp_move<0xB1, 0xF>(v, v);
  }
}
// (every lane of the wave must be running where these are called; the workgroup is one-dimensional)
template <int OFF> __device__ __forceinline__ float lane_xor(float v) { return __uint_as_float(lane_xor_bits<OFF>(__float_as_uint(v))); }
template <int OFF> __device__ __forceinline__ int lane_xor(int v) { return (int)lane_xor_bits<OFF>((unsigned)v); }

// ---- wave64 reductions in a fixed order ----------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
  v += lane_xor<32>(v);
  v += lane_xor<16>(v);
  v += lane_xor<8>(v);
  v += lane_xor<4>(v);
  v += lane_xor<2>(v);
  v += lane_xor<1>(v);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
  v = fmaxf(v, lane_xor<32>(v));
  v = fmaxf(v, lane_xor<16>(v));
  v = fmaxf(v, lane_xor<8>(v));
  v = fmaxf(v, lane_xor<4>(v));
  v = fmaxf(v, lane_xor<2>(v));
  v = fmaxf(v, lane_xor<1>(v));
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
