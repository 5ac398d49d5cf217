// Device helpers of the fp8 activation cast shared by the row kernels and the gate kernel
// (fp8_linear, /root/reference/comfy/ops.py:337-343).
#pragma once
#include "common.h"
#include "numfmt.h"

struct HdmoeScalePtrs {
  const float* p[HDMOE_MAX_EXPERTS];
};

#if defined(__HIPCC__)
// inv < 0 selects the scale_input-is-None rule (clamp to +-448, scale 1).
__device__ __forceinline__ float hdmoe_q_pre(float v, float inv) {
  if (inv < 0.0f) return v < -448.0f ? -448.0f : (v > 448.0f ? 448.0f : v);
  return hdmoe_dev_round_bf16(v * inv);  // bf16 tensor times bf16 scalar, rounded to bf16
}

// two bf16 values (one packed word) -> two e4m3fn bytes in the low 16 bits
__device__ __forceinline__ uint32_t hdmoe_q_2(uint32_t u, float inv) {
  return hdmoe_dev_pack_e4m3fn(hdmoe_q_pre(__uint_as_float(u << 16), inv),
                               hdmoe_q_pre(__uint_as_float(u & 0xffff0000u), inv));
}

// eight bf16 values -> eight e4m3fn bytes
__device__ __forceinline__ uint2 hdmoe_q_8(const uint4& v, float inv) {
  uint2 o;
  o.x = hdmoe_q_2(v.x, inv) | (hdmoe_q_2(v.y, inv) << 16);
  o.y = hdmoe_q_2(v.z, inv) | (hdmoe_q_2(v.w, inv) << 16);
  return o;
}

// (1.0 / scale_input).to(bfloat16) as fp32; NULL pointer -> clamp rule marker
__device__ __forceinline__ float hdmoe_q_inv_scale(const float* s) {
  if (s == nullptr) return -1.0f;
  return hdmoe_dev_round_bf16(__fdiv_rn(1.0f, *s));
}
#endif
