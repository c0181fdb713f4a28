// Seeded normal values from a counter: element i of a tensor depends on (key, i) alone, so a tensor
// is the same whoever makes it, in whatever pieces, on the GPU (here) or on the CPU
// (weights/counter_normal.py, the same operations on numpy arrays).
//
//   z       = splitmix64's (i / 2 + 1)-th output from state `key`: one draw for elements 2p and 2p + 1
//   u1      = ((z >> 40) + 1) / 2^24 in (0, 1],  u2 = ((z >> 8) & 0xFFFFFF) / 2^24 in [0, 1)
//   normals = sqrt(-2 ln u1) * cos(2 pi u2) for the even element, * sin(2 pi u2) for the odd one   (Box-Muller)
//   value   = normal * scale + shift, rounded once to the output type
//
// ln and cos are polynomials of float32 additions, multiplications, one division and one square
// root, each rounded on its own (no fused multiply-add: `fp contract(off)`), in one fixed order:
// every operation is IEEE's correctly rounded one on both sides, so the bits agree.
#include "common.h"

namespace xi {

// the two normal values of pair p (elements 2p and 2p + 1)
__device__ __forceinline__ void counter_normal_pair(uint64_t key, uint64_t pair, float& even, float& odd) {
#pragma clang fp contract(off)
  uint64_t z = key + (pair + 1) * 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  z = z ^ (z >> 31);
  const uint32_t k = (uint32_t)(z >> 40) + 1u;          // 1 .. 2^24
  const uint32_t b = (uint32_t)(z >> 8) & 0xFFFFFFu;    // 0 .. 2^24 - 1
  // ln(k / 2^24) = (e - 24) ln 2 + ln m, k = m 2^e, m in [1/sqrt 2, sqrt 2)
  int e = 31 - __clz((int)k);
  float m = (float)k * __uint_as_float((uint32_t)(127 - e) << 23);   // exact: k has at most 24 bits
  if (m > 1.41421354f) {
    m = m * 0.5f;
    e += 1;
  }
  const float s = (m - 1.0f) / (m + 1.0f);
  const float s2 = s * s;
  float p = 0.111111112f;
  p = p * s2 + 0.142857149f;
  p = p * s2 + 0.200000003f;
  p = p * s2 + 0.333333343f;
  p = p * s2 + 1.0f;
  const float ln_u = (float)(e - 24) * 0.693147182f + (2.0f * s) * p;
  const float radius = sqrtf(-2.0f * ln_u);
  // cos(2 pi b / 2^24): the two top bits of b name the quarter turn, the rest an angle t in [0, pi / 2)
  const uint32_t quarter = b >> 22;
  const float t = (float)(b & 0x3FFFFFu) * 2.38418579e-07f * 1.57079637f;
  const float t2 = t * t;
  float sn = -2.50521084e-08f;
  sn = sn * t2 + 2.75573188e-06f;
  sn = sn * t2 + -1.98412701e-04f;
  sn = sn * t2 + 8.33333377e-03f;
  sn = sn * t2 + -1.66666672e-01f;
  sn = sn * t2 + 1.0f;
  sn = sn * t;
  float cs = 2.08767559e-09f;
  cs = cs * t2 + -2.75573192e-07f;
  cs = cs * t2 + 2.48015876e-05f;
  cs = cs * t2 + -1.38888892e-03f;
  cs = cs * t2 + 4.16666679e-02f;
  cs = cs * t2 + -0.5f;
  cs = cs * t2 + 1.0f;
  const float c = quarter == 0 ? cs : quarter == 1 ? -sn : quarter == 2 ? -cs : sn;
  const float sv = quarter == 0 ? sn : quarter == 1 ? cs : quarter == 2 ? -sn : -cs;
  even = radius * c;
  odd = radius * sv;
}

template <typename T>
__global__ void __launch_bounds__(256) counter_normal_kernel(T* __restrict__ out, uint64_t n, uint64_t first,
                                                             uint64_t key, float scale, float shift) {
#pragma clang fp contract(off)
  // a thread a pair: elements 2p and 2p + 1 of the stream, those of them that lie in [first, first + n)
  const uint64_t p0 = first >> 1, pairs = ((first + n + 1) >> 1) - p0;
  for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < pairs; i += (uint64_t)gridDim.x * 256) {
    float a, b;
    counter_normal_pair(key, p0 + i, a, b);
    const uint64_t e = 2 * (p0 + i);
    if (e >= first) out[e - first] = from_float<T>(a * scale + shift);
    if (e + 1 >= first && e + 1 < first + n) out[e + 1 - first] = from_float<T>(b * scale + shift);
  }
}

}  // namespace xi

// out[i] = normal(key, first + i) * scale + shift for i < n; out is float32 (dtype 0) or bfloat16 (1).
extern "C" int xi_counter_normal(void* out, unsigned long long n, unsigned long long first, unsigned long long key,
                                 float scale, float shift, int dtype, hipStream_t stream) {
  using namespace xi;
  XI_CHECK(out != nullptr || n == 0, "counter_normal: no output");
  XI_CHECK(dtype == kF32 || dtype == kBF16, "counter_normal: dtype %d is neither float32 nor bfloat16", dtype);
  if (n == 0) return 0;
  const unsigned long long want = (n / 2 + 256) / 256;
  const unsigned grid = (unsigned)(want < 65536ull ? want : 65536ull);
  if (dtype == kF32)
    counter_normal_kernel<float><<<grid, 256, 0, stream>>>((float*)out, n, first, key, scale, shift);
  else
    counter_normal_kernel<bf16><<<grid, 256, 0, stream>>>((bf16*)out, n, first, key, scale, shift);
  XI_LAUNCH_CHECK("counter_normal");
  return 0;
}
