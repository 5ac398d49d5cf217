// Device helpers of the fp8 activation cast shared by the row kernels and the gate kernel
// (fp8_linear, /root/reference/comfy/ops.py:337-343).
#pragma once
#include "common.h"
#include "numfmt.h"

struct HdmoeScalePtrs {
  const float* p[HDMOE_MAX_EXPERTS];
};

#if defined(__HIPCC__)
// All helpers take inv = (1.0 / scale_input).to(bfloat16), or a negative value for the scale_input-is-None rule
// (clamp to +-448, scale 1). inv must be the same in every lane of the wave; pass it through hdmoe_q_uniform
// once so that the branches on it are scalar.
__device__ __forceinline__ float hdmoe_q_uniform(float inv) {
  return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(inv)));
}

__device__ __forceinline__ float hdmoe_q_pre(float v, float inv) {
  if (inv < 0.0f) return v < -448.0f ? -448.0f : (v > 448.0f ? 448.0f : v);
  return hdmoe_dev_round_bf16(v * inv);  // bf16 tensor times bf16 scalar, rounded to bf16
}

// two bf16 values (one packed word) -> two e4m3fn bytes in the low 16 bits
__device__ __forceinline__ uint32_t hdmoe_q_2(uint32_t u, float inv) {
  return hdmoe_dev_pack_e4m3fn(hdmoe_q_pre(__uint_as_float(u << 16), inv),
                               hdmoe_q_pre(__uint_as_float(u & 0xffff0000u), inv));
}

// eight bf16 values -> eight e4m3fn bytes. A scale of exactly 1 casts the packed pairs as they are (x * 1 rounded
// to bf16 is x); otherwise the products are rounded to bf16 as packed pairs and cast from those.
__device__ __forceinline__ uint2 hdmoe_q_8(const uint4& v, float inv) {
  const uint32_t w[4] = {v.x, v.y, v.z, v.w};
  if (inv == 1.0f) return make_uint2(hdmoe_dev_pack4_e4m3fn_bf16(w[0], w[1]), hdmoe_dev_pack4_e4m3fn_bf16(w[2], w[3]));
  float f[8];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = __uint_as_float(w[j] << 16);
    f[2 * j + 1] = __uint_as_float(w[j] & 0xffff0000u);
  }
  if (inv < 0.0f) {
#pragma unroll
    for (int j = 0; j < 8; ++j) f[j] = f[j] < -448.0f ? -448.0f : (f[j] > 448.0f ? 448.0f : f[j]);
    return make_uint2(hdmoe_dev_pack4_e4m3fn(f[0], f[1], f[2], f[3]), hdmoe_dev_pack4_e4m3fn(f[4], f[5], f[6], f[7]));
  }
  uint32_t p[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) p[j] = hdmoe_dev_pack_bf16(f[2 * j] * inv, f[2 * j + 1] * inv);
  return make_uint2(hdmoe_dev_pack4_e4m3fn_bf16(p[0], p[1]), hdmoe_dev_pack4_e4m3fn_bf16(p[2], p[3]));
}

// (1.0 / scale_input).to(bfloat16) as fp32; NULL pointer -> clamp rule marker
__device__ __forceinline__ float hdmoe_q_inv_scale(const float* s) {
  if (s == nullptr) return -1.0f;
  return hdmoe_dev_round_bf16(__fdiv_rn(1.0f, *s));
}
#endif
