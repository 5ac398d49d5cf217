// Host-side export of the integer bf16 / e4m3fn conversions in comfyui_amd/csrc/numfmt.h, so the CPU
// tests can pin them against torch exhaustively (the HIP kernels use the same header).
#include "../comfyui_amd/csrc/numfmt.h"
extern "C" {
void t_f32_to_bf16(const float* in, uint16_t* out, long n) { for (long i = 0; i < n; ++i) out[i] = hdmoe_f32_to_bf16(in[i]); }
void t_f32_to_e4m3fn(const float* in, uint8_t* out, long n) { for (long i = 0; i < n; ++i) out[i] = hdmoe_f32_to_e4m3fn(in[i]); }
void t_e4m3fn_to_f32(const uint8_t* in, float* out, long n) { for (long i = 0; i < n; ++i) out[i] = hdmoe_e4m3fn_to_f32(in[i]); }
}
