// Measurement support, not part of the feed-forward: the rate at which the matrix cores of this GPU retire the fp8
// MFMA instructions the GEMM kernels are built on, with operands that stay in registers (no LDS, no memory), on
// operand bytes the caller supplies (zeros, or e4m3fn casts of N(0,1) values: the rate depends on the data, because
// the clock the device sustains under the instruction does). bench.py --aux-kernels runs it to put a measured ceiling
// beside the published peak. Built into its own library (libhdmoe_probe.so); nothing in libhdmoe.so uses it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

constexpr int THREADS = 512;   // 8 waves per block, two per SIMD, as the GEMM kernels run
constexpr int NACC = 10;       // independent accumulators per wave (the 320-token tile has 2 x 5 per K slice)

// FORM 0: v_mfma_f32_32x32x64_f8f6f4, FORM 1: v_mfma_f32_16x16x128_f8f6f4 (same FLOP per instruction pair: one
// 32x32x64 = 131072 FLOP, one 16x16x128 = 65536 FLOP)
template <int FORM>
__global__ __launch_bounds__(THREADS) void mfma_rate_kernel(const v8i* __restrict__ operands, int iters,
                                                            long long* __restrict__ ticks, float* __restrict__ sink) {
  // two operand fragments per lane: 32 bytes each, from the caller's buffer
  const size_t i = ((size_t)blockIdx.x * THREADS + threadIdx.x) * 2;
  const v8i a = operands[i], b = operands[i + 1];
  float total = 0.0f;
  const long long c0 = clock64(), w0 = wall_clock64();
  if constexpr (FORM == 0) {
    v16f acc[NACC];
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
      for (int k = 0; k < 16; ++k) acc[j][k] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < NACC; ++j)
        acc[j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[j], 0, 0, 0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
      for (int k = 0; k < 16; ++k) total += acc[j][k];
  } else {
    v4f acc[NACC];
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) acc[j][k] = 0.0f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int j = 0; j < NACC; ++j)
        acc[j] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[j], 0, 0, 0, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < NACC; ++j)
#pragma unroll
      for (int k = 0; k < 4; ++k) total += acc[j][k];
  }
  const long long c1 = clock64(), w1 = wall_clock64();
  if (total == 12345.678f) sink[0] = total;   // keeps the accumulators alive
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    ticks[0] = c1 - c0;   // s_memtime ticks
    ticks[1] = w1 - w0;   // constant-rate counter ticks (wall_clock64)
  }
}

}  // namespace

// FLOP of one launch: blocks * 8 waves * iters * NACC * (131072 or 65536).
// operands: blocks * 512 * 64 bytes on the device; ticks: 2 x int64 on the device; sink: one float on the device.
extern "C" int hdmoe_probe_mfma_fp8(int form, const void* operands, int blocks, int iters, long long* ticks, float* sink,
                                    void* stream) {
  if (operands == nullptr || ticks == nullptr || sink == nullptr || blocks < 1 || iters < 1 || form < 0 || form > 1) return -2;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (form == 0)
    hipLaunchKernelGGL(mfma_rate_kernel<0>, dim3(blocks), dim3(THREADS), 0, s, static_cast<const v8i*>(operands), iters, ticks, sink);
  else
    hipLaunchKernelGGL(mfma_rate_kernel<1>, dim3(blocks), dim3(THREADS), 0, s, static_cast<const v8i*>(operands), iters, ticks, sink);
  return hipGetLastError() == hipSuccess ? 0 : -4;
}

extern "C" int hdmoe_probe_accumulators(void) { return NACC; }
extern "C" int hdmoe_probe_wall_clock_khz(void) {
  int khz = 0;
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess) return 0;
  if (hipDeviceGetAttribute(&khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess) return 0;
  return khz;
}
