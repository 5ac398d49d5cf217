// Bit-level bf16 and float8_e4m3fn conversions shared by the HIP kernels (device)
// and the host-side self checks. Plain integer arithmetic on IEEE-754 fp32 bit
// patterns, so host and device produce identical bytes.
//
// float8_e4m3fn: 1 sign, 4 exponent (bias 7), 3 mantissa bits; no infinities;
// 0x7F / 0xFF are NaN; largest finite value 448. The encode below is
// round-to-nearest-even WITHOUT saturation: |v| > 464 (the midpoint between 448
// and the would-be 480) becomes NaN, exactly what `tensor.to(torch.float8_e4m3fn)`
// produces and therefore what the reference's fp8_linear feeds torch._scaled_mm
// (/root/reference/comfy/ops.py:337-343).
#pragma once
#include <stdint.h>
#include <string.h>

#if defined(__HIPCC__)
#define HDMOE_HD __host__ __device__ __forceinline__
#else
#define HDMOE_HD static inline
#endif

HDMOE_HD uint32_t hdmoe_f32_bits(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __float_as_uint(f);
#else
  uint32_t u;
  memcpy(&u, &f, 4);
  return u;
#endif
}

HDMOE_HD float hdmoe_bits_f32(uint32_t u) {
#if defined(__HIP_DEVICE_COMPILE__)
  return __uint_as_float(u);
#else
  float f;
  memcpy(&f, &u, 4);
  return f;
#endif
}

// bf16 <-> fp32. Encode is round-to-nearest-even; NaN stays NaN (quiet bit forced).
HDMOE_HD float hdmoe_bf16_to_f32(uint16_t h) { return hdmoe_bits_f32((uint32_t)h << 16); }

HDMOE_HD uint16_t hdmoe_f32_to_bf16(float f) {
  uint32_t u = hdmoe_f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

// fp32 value rounded to the nearest bf16 and returned as fp32.
HDMOE_HD float hdmoe_round_bf16(float f) { return hdmoe_bf16_to_f32(hdmoe_f32_to_bf16(f)); }

HDMOE_HD float hdmoe_e4m3fn_to_f32(uint8_t b) {
  uint32_t sign = (uint32_t)(b & 0x80u) << 24;
  uint32_t e = (b >> 3) & 0xfu;
  uint32_t m = b & 7u;
  if (e == 0xfu && m == 7u) return hdmoe_bits_f32(sign | 0x7fc00000u);
  if (e == 0u) {
    // subnormal: m * 2^-9, exact in fp32
    float v = (float)m * 0.001953125f;
    return hdmoe_bits_f32(hdmoe_f32_bits(v) | sign);
  }
  return hdmoe_bits_f32(sign | ((e + 120u) << 23) | (m << 20));
}

HDMOE_HD uint8_t hdmoe_f32_to_e4m3fn(float f) {
  uint32_t u = hdmoe_f32_bits(f);
  uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
  uint32_t a = u & 0x7fffffffu;
  if (a >= 0x43f00000u) return (uint8_t)(sign | 0x7fu);  // >= 480, inf, NaN
  if (a < 0x3c800000u) {
    // below the smallest normal 2^-6: align the ulp to 2^-9 by adding 2^14
    // (fp32 ulp at 2^14 is 2^-9); the hardware add performs the RNE.
    float t = hdmoe_bits_f32(a) + 16384.0f;
    return (uint8_t)(sign | (uint8_t)(hdmoe_f32_bits(t) - 0x46800000u));
  }
  a += 0x7ffffu + ((a >> 20) & 1u);  // RNE on the 20 dropped mantissa bits
  // exponent field rebias 127 -> 7; a carry out of the mantissa bumps the exponent,
  // and 0x7F (would-be 480) is the NaN pattern, which is the no-saturation rule.
  return (uint8_t)(sign | (uint8_t)((a >> 20) - 0x3c0u));
}

#if defined(__HIPCC__)
// ---- device-only fast paths on the gfx950 conversion instructions --------------------
// v_cvt_pk_bf16_f32 rounds to nearest even; v_cvt_pk_fp8_f32 converts two fp32 values to
// OCP e4m3fn. Both are checked bit for bit against the integer versions above by the GPU
// tests (every bf16 input pattern for the fp8 cast, torch's own bf16 arithmetic for the
// bf16 rounding).
typedef __bf16 hdmoe_bf16x2 __attribute__((ext_vector_type(2)));
typedef float hdmoe_f32x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t hdmoe_dev_pack_bf16(float lo, float hi) {
  hdmoe_f32x2 v = {lo, hi};
  hdmoe_bf16x2 b = __builtin_convertvector(v, hdmoe_bf16x2);
  return *reinterpret_cast<uint32_t*>(&b);
}

__device__ __forceinline__ float hdmoe_dev_round_bf16(float f) {
  return __uint_as_float(hdmoe_dev_pack_bf16(f, 0.0f) << 16);
}

// ---- the two 16-bit activation formats as one interface ------------------------------------------------
// A kernel templated on the format reads packed pairs with lo()/hi(), rounds an fp32 value to the format with
// round() and packs two with pack(); all conversions round to nearest even (v_cvt_f16_f32 follows the wave's
// rounding mode, which no kernel here changes from the default). fp16 overflows to infinity and keeps its
// subnormals, as torch's conversion does.
typedef _Float16 hdmoe_f16x2 __attribute__((ext_vector_type(2)));

struct HdmoeBf16 {
  static __device__ __forceinline__ float lo(uint32_t u) { return __uint_as_float(u << 16); }
  static __device__ __forceinline__ float hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
  static __device__ __forceinline__ uint32_t pack(float a, float b) { return hdmoe_dev_pack_bf16(a, b); }
  static __device__ __forceinline__ float round(float f) { return hdmoe_dev_round_bf16(f); }
};

struct HdmoeF16 {
  static __device__ __forceinline__ float lo(uint32_t u) { return (float)(*reinterpret_cast<hdmoe_f16x2*>(&u))[0]; }
  static __device__ __forceinline__ float hi(uint32_t u) { return (float)(*reinterpret_cast<hdmoe_f16x2*>(&u))[1]; }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    hdmoe_f16x2 h = {(_Float16)a, (_Float16)b};
    return *reinterpret_cast<uint32_t*>(&h);
  }
  static __device__ __forceinline__ float round(float f) { return (float)(_Float16)f; }
};

// e4m3fn conversion with the no-saturation rule (beyond the rounding midpoint above 448 -> NaN, 0x7F):
// v_cvt_pk_fp8_f32 follows it when the FP16_OVFL bit of the wave's MODE register is clear and saturates to 448
// when it is set. A wave starts with the bit its kernel descriptor holds (.amdhsa_fp16_overflow), which is 0 for
// every kernel built from these sources, and no kernel here changes it (writing MODE in the GEMM kernel also cost
// it 85 spilled registers). Checked bit for bit over every bf16 input pattern by the GPU tests.

// e4m3fn bytes of (a, b) in the low 16 bits
__device__ __forceinline__ uint32_t hdmoe_dev_pack_e4m3fn(float a, float b) {
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false) & 0xffffu;
}

// e4m3fn bytes of four bf16 values given as two packed words (p01 = values 0 and 1, value 0 in the low half):
// v_cvt_scalef32_pk_fp8_bf16 with a scale of 1 converts a bf16 pair without unpacking it and follows the same
// no-saturation rule (checked over every bf16 pattern on the device).
typedef short hdmoe_i16x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t hdmoe_dev_pack4_e4m3fn_bf16(uint32_t p01, uint32_t p23) {
  hdmoe_i16x2 r = {0, 0};
  r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r, *reinterpret_cast<hdmoe_bf16x2*>(&p01), 1.0f, false);
  r = __builtin_amdgcn_cvt_scalef32_pk_fp8_bf16(r, *reinterpret_cast<hdmoe_bf16x2*>(&p23), 1.0f, true);
  return *reinterpret_cast<uint32_t*>(&r);
}

// e4m3fn bytes of (a, b, c, d), a in the lowest byte
__device__ __forceinline__ uint32_t hdmoe_dev_pack4_e4m3fn(float a, float b, float c, float d) {
  const int lo = __builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
  return (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(c, d, lo, true);
}
#endif
