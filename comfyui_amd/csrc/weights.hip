// Weight-side maintenance for scaled-fp8 Linears: stochastic rounding of a patched weight back to
// float8_e4m3fn, fused with the division by scale_weight
// (/root/reference/comfy/ops.py:419-426 set_weight -> /root/reference/comfy/float.py:14-67).
//
// As in the reference the value is first rounded to float16; it then lands on one of its two e4m3fn neighbours,
// the upper one with probability equal to its fractional position between them (position + u floored, u uniform
// in [0,1)), magnitudes of 448 and more saturate to +-448, zero stays zero. The uniform numbers are not torch's:
// element i takes word (i & 3) of Philox4x32-10(counter = i >> 2, key = seed), 24 bits of it, so the result depends
// only on (value, seed, i).
#include <hip/hip_fp16.h>

#include "common.h"
#include "numfmt.h"
#include "philox.h"

namespace {

constexpr int THREADS = 256;

// |value| already rounded to float16 (as fp32), one 32-bit random word -> e4m3fn code without sign
__device__ __forceinline__ uint32_t sr_code(float a, uint32_t rnd) {
  if (!(a < 448.0f)) return a != a ? 0x7fu : 0x7eu;  // NaN stays NaN; 448 and beyond (inf too) saturate
  if (a == 0.0f) return 0u;
  const float u = (float)(rnd >> 8) * 0x1p-24f;
  const int e = (int)((__float_as_uint(a) >> 23) & 0xffu) - 127;  // floor(log2 a): a float16 value is normal in fp32
  if (e >= -6) {
    // normal binade 2^e * (1 + k/8): position in eighths
    const float pos = (a * __uint_as_float((uint32_t)(127 - e) << 23) - 1.0f) * 8.0f;
    const uint32_t k = (uint32_t)(pos + u);                          // 0..8, 8 carries into the next binade
    const uint32_t code = ((uint32_t)(e + 7) << 3) + k;
    return code > 0x7eu ? 0x7eu : code;
  }
  // subnormal binade: steps of 2^-9
  return (uint32_t)(a * 512.0f + u);                                  // 0..8, 8 is the smallest normal
}

template <typename SRC>
__device__ __forceinline__ float load_scaled(const SRC* src, long i, float s);

template <>
__device__ __forceinline__ float load_scaled<float>(const float* src, long i, float s) {
  return __fdiv_rn(src[i], s);
}

// bf16 weights: the reference divides two bf16 tensors, so the scale and the quotient are rounded to bf16
template <>
__device__ __forceinline__ float load_scaled<uint16_t>(const uint16_t* src, long i, float s) {
  return hdmoe_round_bf16(__fdiv_rn(hdmoe_bf16_to_f32(src[i]), hdmoe_round_bf16(s)));
}

template <typename SRC>
__global__ __launch_bounds__(THREADS) void stochastic_round_kernel(const SRC* __restrict__ src, long n,
                                                                   const float* __restrict__ scale, uint32_t seed_lo,
                                                                   uint32_t seed_hi, uint8_t* __restrict__ out) {
  const float s = scale ? *scale : 1.0f;
  const uint32_t key[2] = {seed_lo, seed_hi};
  const long groups = (n + 3) / 4;
  for (long g = (long)blockIdx.x * THREADS + threadIdx.x; g < groups; g += (long)gridDim.x * THREADS) {
    const uint32_t ctr[4] = {(uint32_t)g, (uint32_t)((uint64_t)g >> 32), 0u, 0u};
    uint32_t r[4];
    hdmoe_philox4x32_10(ctr, key, r);
    uint32_t packed = 0;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const long i = g * 4 + j;
      if (i < n) {
        const float x = __half2float(__float2half_rn(load_scaled<SRC>(src, i, s)));
        // an exact zero stays +0 (the reference multiplies by sign(0) = 0); a value rounded down to zero keeps its sign
        const uint32_t code = x == 0.0f ? 0u : (sr_code(__builtin_fabsf(x), r[j]) | ((__float_as_uint(x) >> 24) & 0x80u));
        packed |= code << (8 * j);
      }
    }
    if (g * 4 + 3 < n) {
      *reinterpret_cast<uint32_t*>(out + g * 4) = packed;
    } else {
      for (int j = 0; g * 4 + j < n; ++j) out[g * 4 + j] = (uint8_t)(packed >> (8 * j));
    }
  }
}

}  // namespace

extern "C" int hdmoe_stochastic_round_e4m3fn(int src_dtype, const void* src, int64_t n, const float* scale_dev,
                                             uint64_t seed, void* out_e4m3fn, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(src);
  HDMOE_REQUIRE_PTR(out_e4m3fn);
  if (n < 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_stochastic_round_e4m3fn: n=%lld", (long long)n);
  if (src_dtype != HDMOE_SRC_BF16 && src_dtype != HDMOE_SRC_F32)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_stochastic_round_e4m3fn: src_dtype=%d is neither HDMOE_SRC_BF16 nor HDMOE_SRC_F32",
                      src_dtype);
  if (((uintptr_t)out_e4m3fn & 3u) != 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_stochastic_round_e4m3fn: output must be 4-byte aligned");
  if (n == 0) return HDMOE_OK;
  const long groups = (n + 3) / 4;
  long blocks = (groups + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 16) blocks = HDMOE_NUM_CU * 16;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint32_t lo = (uint32_t)seed, hi = (uint32_t)(seed >> 32);
  if (src_dtype == HDMOE_SRC_F32)
    hipLaunchKernelGGL(stochastic_round_kernel<float>, dim3((int)blocks), dim3(THREADS), 0, s,
                       static_cast<const float*>(src), (long)n, scale_dev, lo, hi, static_cast<uint8_t*>(out_e4m3fn));
  else
    hipLaunchKernelGGL(stochastic_round_kernel<uint16_t>, dim3((int)blocks), dim3(THREADS), 0, s,
                       static_cast<const uint16_t*>(src), (long)n, scale_dev, lo, hi, static_cast<uint8_t*>(out_e4m3fn));
  return hdmoe_check_launch("hdmoe_stochastic_round_e4m3fn");
}
