// Bandwidth-bound row kernels around the GEMMs: activation quantisation (with and
// without the dispatch gather), the bf16 gather, SiLU*mul for the unfused path and
// the weighted combine. One wavefront per row; a lane moves 8 elements (16 bytes of
// bf16) per 512-element chunk, so every load instruction of a wave covers 1 KiB of
// one row.
#include "common.h"
#include "numfmt.h"
#include "quant.h"

namespace {

constexpr int THREADS = 256;
constexpr int WAVES = THREADS / 64;

typedef HdmoeScalePtrs ScalePtrs;

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) { return hdmoe_dev_pack_bf16(lo, hi); }
__device__ __forceinline__ float round_bf16(float f) { return hdmoe_dev_round_bf16(f); }
__device__ __forceinline__ uint2 quant8(const uint4& v, float inv) { return hdmoe_q_8(v, inv); }
__device__ __forceinline__ float inv_scale(const float* s) { return hdmoe_q_uniform(hdmoe_q_inv_scale(s)); }

// scale_in_also: scale_input of a second Linear that reads this cast (w3 beside w1). Where its cast factor differs the
// one cast cannot serve both: the rows are written as NaN (products with a NaN factor).
__global__ __launch_bounds__(THREADS) void quant_rows_kernel(const uint4* __restrict__ x, long rows, int row16,
                                                             const float* scale_in, const float* scale_in_also,
                                                             uint2* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const long wave = (long)blockIdx.x * WAVES + (threadIdx.x >> 6);
  const long nwaves = (long)gridDim.x * WAVES;
  float inv = inv_scale(scale_in);
  if (scale_in_also != scale_in && inv_scale(scale_in_also) != inv) inv = __builtin_nanf("");
  for (long r = wave; r < rows; r += nwaves)
    for (int u = lane; u < row16; u += 64) out[r * row16 + u] = quant8(x[r * row16 + u], inv);
}

// Quantise the rows the expert GEMMs read: sorted rows [0, rows_routed) gather token perm[r]/2 with the
// scale_input of the expert whose segment holds r; rows [rows_routed, rows_total) are the token-order copy for
// the shared expert. Two rows per wave and iteration keep 2 x NCH 16-byte loads per lane in flight.
// NCH * 64 == row16 selects the unrolled path, NCH == 0 the generic one.
template <int NCH>
__global__ __launch_bounds__(THREADS) void quant_dispatch_kernel(const uint4* __restrict__ x,
                                                                 const int32_t* __restrict__ perm,
                                                                 const int32_t* __restrict__ offsets, int rows_routed,
                                                                 int rows_total, int E, int row16, ScalePtrs sp,
                                                                 const float* shared_scale, uint2* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES;
  for (int r0 = wave * 2; r0 < rows_total; r0 += nwaves * 2) {
    long t[2];
    float inv[2];
    bool ok[2];
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int r = r0 + k;
      ok[k] = r < rows_total;
      t[k] = 0;
      inv[k] = 1.0f;
      if (!ok[k]) continue;
      if (r < rows_routed) {
        t[k] = perm[r] / HDMOE_TOPK;
        int e = 0;
        while (e + 1 < E && r >= offsets[e + 1]) ++e;
        inv[k] = inv_scale(sp.p[e]);
      } else {
        t[k] = r - rows_routed;
        inv[k] = inv_scale(shared_scale);
      }
    }
    if constexpr (NCH > 0) {
      uint4 v[2][NCH];
#pragma unroll
      for (int k = 0; k < 2; ++k)
#pragma unroll
        for (int c = 0; c < NCH; ++c) v[k][c] = ok[k] ? x[t[k] * row16 + c * 64 + lane] : make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int k = 0; k < 2; ++k)
        if (ok[k]) {
#pragma unroll
          for (int c = 0; c < NCH; ++c) out[(long)(r0 + k) * row16 + c * 64 + lane] = quant8(v[k][c], inv[k]);
        }
    } else {
#pragma unroll
      for (int k = 0; k < 2; ++k)
        if (ok[k])
          for (int u = lane; u < row16; u += 64) out[(long)(r0 + k) * row16 + u] = quant8(x[t[k] * row16 + u], inv[k]);
    }
  }
}

__global__ __launch_bounds__(THREADS) void permute_rows_kernel(const uint4* __restrict__ x,
                                                               const int32_t* __restrict__ perm, int rows, int row16,
                                                               uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES;
  for (int r = wave; r < rows; r += nwaves) {
    const long t = perm[r] / HDMOE_TOPK;
    for (int u = lane; u < row16; u += 64) out[(long)r * row16 + u] = x[t * row16 + u];
  }
}

// bf16( bf16(silu(a)) * b ); silu evaluated in fp32 as a / (1 + exp(-a))
__device__ __forceinline__ float silu_mul1(float a, float b) {
  const float s = round_bf16(a * __builtin_amdgcn_rcpf(1.0f + __expf(-a)));
  return s * b;
}

__global__ __launch_bounds__(THREADS) void silu_mul_kernel(const uint4* __restrict__ a, const uint4* __restrict__ b,
                                                           long n16, uint4* __restrict__ out) {
  const long stride = (long)gridDim.x * THREADS;
  for (long i = (long)blockIdx.x * THREADS + threadIdx.x; i < n16; i += stride) {
    const uint4 va = a[i], vb = b[i];
    uint4 o;
    o.x = pack_bf16(silu_mul1(bf16_lo(va.x), bf16_lo(vb.x)), silu_mul1(bf16_hi(va.x), bf16_hi(vb.x)));
    o.y = pack_bf16(silu_mul1(bf16_lo(va.y), bf16_lo(vb.y)), silu_mul1(bf16_hi(va.y), bf16_hi(vb.y)));
    o.z = pack_bf16(silu_mul1(bf16_lo(va.z), bf16_lo(vb.z)), silu_mul1(bf16_hi(va.z), bf16_hi(vb.z)));
    o.w = pack_bf16(silu_mul1(bf16_lo(va.w), bf16_lo(vb.w)), silu_mul1(bf16_hi(va.w), bf16_hi(vb.w)));
    out[i] = o;
  }
}

// F.gelu (erf form) of a bf16 tensor, evaluated in fp32 and rounded once
// (/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:14-26), for projections whose Linear is not the plain bf16 one.
__device__ __forceinline__ float gelu1(float h) { return 0.5f * h * (1.0f + erff(h * 0.70710678118654752440f)); }

template <class A>  // HdmoeBf16 or HdmoeF16: the tensor's element format
__global__ __launch_bounds__(THREADS) void gelu_kernel(const uint4* __restrict__ x, int64_t n8, uint4* __restrict__ out) {
  for (int64_t i = blockIdx.x * (int64_t)THREADS + threadIdx.x; i < n8; i += (int64_t)gridDim.x * THREADS) {
    const uint4 v = x[i];
    uint4 o;
    o.x = A::pack(gelu1(A::lo(v.x)), gelu1(A::hi(v.x)));
    o.y = A::pack(gelu1(A::lo(v.y)), gelu1(A::hi(v.y)));
    o.z = A::pack(gelu1(A::lo(v.z)), gelu1(A::hi(v.z)));
    o.w = A::pack(gelu1(A::lo(v.w)), gelu1(A::hi(v.w)));
    out[i] = o;
  }
}

// topk_weight / (topk_weight.sum(-1, keepdim=True) + 1e-20) on a [T, 2] bf16 tensor
// (/root/reference/comfy/ldm/hidream/model.py:277-280): the sum is rounded to bf16, the scalar is added in fp32 and the
// result rounded to bf16 again, then each quotient is rounded to bf16, as the three torch ops do.
__global__ __launch_bounds__(THREADS) void renorm_top2_kernel(const uint32_t* __restrict__ w, int T,
                                                              uint32_t* __restrict__ out) {
  for (int t = blockIdx.x * THREADS + threadIdx.x; t < T; t += gridDim.x * THREADS) {
    const uint32_t v = w[t];
    const float w0 = bf16_lo(v), w1 = bf16_hi(v);
    const float sum = __uint_as_float(pack_bf16(w0 + w1, 0.0f) << 16);
    const float den = __uint_as_float(pack_bf16(sum + 1e-20f, 0.0f) << 16);
    out[t] = pack_bf16(__fdiv_rn(w0, den), __fdiv_rn(w1, den));
  }
}

// (y.view(T,2,D) * w.unsqueeze(-1)).sum(1) + shared at bf16
// (/root/reference/comfy/ldm/hidream/model.py:319,324): each product is rounded to
// bf16, the two-term sum is formed in fp32 and rounded, then the shared row is added
// and the result rounded again.
// Optional block epilogue on top: bf16( bf16(gate_mlp * .) + residual )  (model.py:432-433, 520-522).
struct CombineExtra {
  const uint4* gate;      // [B, D] bf16 or NULL
  const uint4* residual;  // [T, D] bf16 (only read when gate != NULL)
  int tokens_per_batch;
};

// A: the element format of every tensor of the call (HdmoeBf16 or HdmoeF16); each "bf16(...)" above is a rounding to it.
template <class A>
__device__ __forceinline__ float comb1(float y0, float y1, float w0, float w1, float sh, bool has_shared, float g,
                                       float res, bool has_gate) {
  // no fused multiply-add: with fp16 the compiler narrows these fp32 operations between two roundings to fp16
  // operations (exact) and would then fuse a product into the following sum, dropping the product's rounding
#pragma clang fp contract(off)
  float s = A::round(A::round(y0 * w0) + A::round(y1 * w1));
  if (has_shared) s = has_gate ? A::round(s + sh) : s + sh;
  if (has_gate) s = A::round(g * s) + res;
  return s;
}

template <class A>
__device__ __forceinline__ uint32_t comb2(uint32_t y0, uint32_t y1, float w0, float w1, uint32_t sh, bool hs, uint32_t g,
                                          uint32_t res, bool hg) {
  return A::pack(comb1<A>(A::lo(y0), A::lo(y1), w0, w1, A::lo(sh), hs, A::lo(g), A::lo(res), hg),
                 comb1<A>(A::hi(y0), A::hi(y1), w0, w1, A::hi(sh), hs, A::hi(g), A::hi(res), hg));
}

template <class A>
__global__ __launch_bounds__(THREADS) void combine_kernel(const uint4* __restrict__ y, const int2* __restrict__ inv_perm,
                                                          const uint32_t* __restrict__ w, const uint4* __restrict__ shared,
                                                          int T, int row16, CombineExtra ex, uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES;
  const bool hs = shared != nullptr;
  const bool hg = ex.gate != nullptr;
  for (int t = wave; t < T; t += nwaves) {
    const int2 r = inv_perm[t];
    const uint32_t wp = w[t];
    const float w0 = A::lo(wp), w1 = A::hi(wp);
    const uint4* y0 = y + (long)r.x * row16;
    const uint4* y1 = y + (long)r.y * row16;
    const long brow = hg ? (long)(t / ex.tokens_per_batch) * row16 : 0;
    for (int u = lane; u < row16; u += 64) {
      const uint4 a = y0[u], b = y1[u];
      uint4 sh = make_uint4(0, 0, 0, 0), g = sh, res = sh;
      if (hs) sh = shared[(long)t * row16 + u];
      if (hg) { g = ex.gate[brow + u]; res = ex.residual[(long)t * row16 + u]; }
      uint4 o;
      o.x = comb2<A>(a.x, b.x, w0, w1, sh.x, hs, g.x, res.x, hg);
      o.y = comb2<A>(a.y, b.y, w0, w1, sh.y, hs, g.y, res.y, hg);
      o.z = comb2<A>(a.z, b.z, w0, w1, sh.z, hs, g.z, res.z, hg);
      o.w = comb2<A>(a.w, b.w, w0, w1, sh.w, hs, g.w, res.w, hg);
      out[(long)t * row16 + u] = o;
    }
  }
}

// The combine of a layer whose down projection was cut along K: the rows come as fp32 partial sums
// [nparts][rows_dyn + T][D] (routed rows in expert order, then the shared expert's), and this kernel first does what
// splitk_reduce_kernel (gemm.hip) does for a row, bf16((sum over the parts in ascending order) * scale of the row's
// Linear), then what combine_kernel does with the three rows of a token. Same operations in the same order as the two
// kernels it replaces, so the same bytes; one launch and one bf16 round trip of the rows less.
struct CombinePartialArgs {
  const float* partial;
  long long part_stride;   // floats between two parts
  HdmoeSplitPlan plan;     // the candidate cuts of the down projection; the entry that ran is chosen as its kernel chose
  int rows_dyn, n_dyn, fp8, has_shared;
  const int32_t* offsets;  // segment bounds of the routed rows, n_dyn + 1 entries
  const float* sw[HDMOE_MAX_EXPERTS + 1];   // scale_weight of the down Linear per expert (fp8); the shared expert is entry n_dyn
  const float* sin[HDMOE_MAX_EXPERTS + 1];  // its scale_input or NULL
};

template <class A>
__global__ __launch_bounds__(THREADS) void combine_partials_kernel(const CombinePartialArgs pa, const int2* __restrict__ inv_perm,
                                                                   const uint32_t* __restrict__ w, int T, int row16,
                                                                   CombineExtra ex, uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES;
  const bool hs = pa.has_shared != 0;
  const bool hg = ex.gate != nullptr;
  const int chunks = (row16 + 63) / 64;   // a wave takes 64 x 8 features of one token at a time
  const int n_out = row16 * 8;
  auto scale_of = [&](int g) -> float { return pa.fp8 ? (pa.sin[g] ? *pa.sin[g] : 1.0f) * *pa.sw[g] : 1.0f; };
  auto group_of = [&](int r) {
    int g = 0;
    while (g + 1 < pa.n_dyn && r >= pa.offsets[g + 1]) ++g;
    return g;
  };
  // the 8 features of row r at column c, as splitk_reduce_kernel leaves them (values of the 16-bit format)
  auto row_vals = [&](int r, int c, float sc, int nparts, float (&v)[8]) {
    const float* src = pa.partial + (size_t)r * n_out + c;
    float4 s0 = *reinterpret_cast<const float4*>(src), s1 = *reinterpret_cast<const float4*>(src + 4);
    for (int p = 1; p < nparts; ++p) {
      const float* q = src + (size_t)p * (size_t)pa.part_stride;
      const float4 t0 = *reinterpret_cast<const float4*>(q), t1 = *reinterpret_cast<const float4*>(q + 4);
      s0.x += t0.x; s0.y += t0.y; s0.z += t0.z; s0.w += t0.w;
      s1.x += t1.x; s1.y += t1.y; s1.z += t1.z; s1.w += t1.w;
    }
    v[0] = A::round(s0.x * sc); v[1] = A::round(s0.y * sc); v[2] = A::round(s0.z * sc); v[3] = A::round(s0.w * sc);
    v[4] = A::round(s1.x * sc); v[5] = A::round(s1.y * sc); v[6] = A::round(s1.z * sc); v[7] = A::round(s1.w * sc);
  };
  const float sc_sh = hs ? scale_of(pa.n_dyn) : 1.0f;
  // which cut the down projection ran with (the same function of the segment bounds as in its kernel)
  int nparts = pa.plan.pd[0], nparts_static = pa.plan.ps[0];
  if (pa.plan.n > 1) {
    // the bounds as one vector load (at most 17 entries), then lane reads
    const int off_lane = lane <= pa.n_dyn ? pa.offsets[lane] : 0;
    int mt_dyn = 0;
    for (int e = 0; e < pa.n_dyn; ++e)
      mt_dyn += (__builtin_amdgcn_readlane(off_lane, e + 1) - __builtin_amdgcn_readlane(off_lane, e) + pa.plan.bm - 1) / pa.plan.bm;
    const int mt_static = hs ? (T + pa.plan.bm - 1) / pa.plan.bm : 0;
    const int idx = hdmoe_plan_pick(pa.plan, mt_dyn, mt_static, n_out / 256);
    nparts = pa.plan.pd[idx];
    nparts_static = pa.plan.ps[idx];
  }
  for (int unit = wave; unit < T * chunks; unit += nwaves) {
    const int t = unit / chunks;
    const int u = (unit - t * chunks) * 64 + lane;
    if (u >= row16) continue;
    const int2 r = inv_perm[t];
    const uint32_t wp = w[t];
    const float w0 = A::lo(wp), w1 = A::hi(wp);
    float y0[8], y1[8], sh[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    row_vals(r.x, u * 8, scale_of(group_of(r.x)), nparts, y0);
    row_vals(r.y, u * 8, scale_of(group_of(r.y)), nparts, y1);
    if (hs) row_vals(pa.rows_dyn + t, u * 8, sc_sh, nparts_static, sh);
    uint4 g = make_uint4(0, 0, 0, 0), res = g;
    if (hg) {
      g = ex.gate[(long)(t / ex.tokens_per_batch) * row16 + u];
      res = ex.residual[(long)t * row16 + u];
    }
    auto two = [&](int i, uint32_t gg, uint32_t rr) {
      return A::pack(comb1<A>(y0[i], y1[i], w0, w1, sh[i], hs, A::lo(gg), A::lo(rr), hg),
                     comb1<A>(y0[i + 1], y1[i + 1], w0, w1, sh[i + 1], hs, A::hi(gg), A::hi(rr), hg));
    };
    uint4 o;
    o.x = two(0, g.x, res.x);
    o.y = two(2, g.y, res.y);
    o.z = two(4, g.z, res.z);
    o.w = two(6, g.w, res.w);
    out[(long)t * row16 + u] = o;
  }
}

// out[t] = bf16( bf16(gate[b] * y[t]) + residual[t] ), b = t / tokens_per_batch: the gate and residual behind a dense
// feed-forward (/root/reference/comfy/ldm/hidream/model.py:519-523, text stream).
__global__ __launch_bounds__(THREADS) void gated_residual_kernel(const uint4* __restrict__ y, const uint4* __restrict__ gate,
                                                                 const uint4* __restrict__ residual, int T, int row16,
                                                                 int tokens_per_batch, uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES;
  auto gr = [](uint32_t g, uint32_t v, uint32_t r) {
    return pack_bf16(round_bf16(bf16_lo(g) * bf16_lo(v)) + bf16_lo(r), round_bf16(bf16_hi(g) * bf16_hi(v)) + bf16_hi(r));
  };
  for (int t = wave; t < T; t += nwaves) {
    const long brow = (long)(t / tokens_per_batch) * row16;
    for (int u = lane; u < row16; u += 64) {
      const uint4 v = y[(long)t * row16 + u], g = gate[brow + u], r = residual[(long)t * row16 + u];
      out[(long)t * row16 + u] = make_uint4(gr(g.x, v.x, r.x), gr(g.y, v.y, r.y), gr(g.z, v.z, r.z), gr(g.w, v.w, r.w));
    }
  }
}

// out = bf16( bf16(src) * bf16(scale) ): the `weight * scale_weight` / `input * scale_weight`
// products of the scaled-fp8 Linear without fp8 matmul (/root/reference/comfy/ops.py:407-410),
// whose operands have already been cast to the compute dtype.
__global__ __launch_bounds__(THREADS) void scale_fp8_to_bf16_kernel(const uint2* __restrict__ src, long n8,
                                                                    const float* scale, uint4* __restrict__ out) {
  const float sc = round_bf16(*scale);
  const long stride = (long)gridDim.x * THREADS;
  for (long i = (long)blockIdx.x * THREADS + threadIdx.x; i < n8; i += stride) {
    const uint2 v = src[i];
    float f[8];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      f[j] = hdmoe_e4m3fn_to_f32((uint8_t)(v.x >> (8 * j))) * sc;
      f[4 + j] = hdmoe_e4m3fn_to_f32((uint8_t)(v.y >> (8 * j))) * sc;
    }
    out[i] = make_uint4(pack_bf16(f[0], f[1]), pack_bf16(f[2], f[3]), pack_bf16(f[4], f[5]), pack_bf16(f[6], f[7]));
  }
}

__global__ __launch_bounds__(THREADS) void scale_bf16_kernel(const uint4* __restrict__ src, long n8, const float* scale,
                                                             uint4* __restrict__ out) {
  const float sc = round_bf16(*scale);
  const long stride = (long)gridDim.x * THREADS;
  for (long i = (long)blockIdx.x * THREADS + threadIdx.x; i < n8; i += stride) {
    const uint4 v = src[i];
    out[i] = make_uint4(pack_bf16(bf16_lo(v.x) * sc, bf16_hi(v.x) * sc), pack_bf16(bf16_lo(v.y) * sc, bf16_hi(v.y) * sc),
                        pack_bf16(bf16_lo(v.z) * sc, bf16_hi(v.z) * sc), pack_bf16(bf16_lo(v.w) * sc, bf16_hi(v.w) * sc));
  }
}

inline int row_blocks(long rows) {
  long b = (rows + WAVES - 1) / WAVES;
  if (b < 1) b = 1;
  if (b > HDMOE_NUM_CU * 16) b = HDMOE_NUM_CU * 16;
  return (int)b;
}

}  // namespace

// One launch for the routed rows [0,2T) and, optionally, the shared expert's token-order rows [2T,3T) of a_fp8.
int hdmoe_launch_quant_dispatch(const void* x_bf16, const int32_t* perm, const int32_t* offsets, int T, int D, int E,
                                const float* const* scale_input, const float* shared_scale, bool with_shared,
                                void* a_fp8, hipStream_t s, const char* what) {
  ScalePtrs sp;
  for (int e = 0; e < HDMOE_MAX_EXPERTS; ++e) sp.p[e] = e < E ? scale_input[e] : nullptr;
  const int rows_routed = T * HDMOE_TOPK;
  const int rows_total = rows_routed + (with_shared ? T : 0);
  const int row16 = D / 8;
  const dim3 grid(row_blocks((rows_total + 1) / 2)), block(THREADS);
  const uint4* xp = static_cast<const uint4*>(x_bf16);
  uint2* op = static_cast<uint2*>(a_fp8);
  if (row16 == 5 * 64)
    hipLaunchKernelGGL(quant_dispatch_kernel<5>, grid, block, 0, s, xp, perm, offsets, rows_routed, rows_total, E, row16,
                       sp, shared_scale, op);
  else
    hipLaunchKernelGGL(quant_dispatch_kernel<0>, grid, block, 0, s, xp, perm, offsets, rows_routed, rows_total, E, row16,
                       sp, shared_scale, op);
  return hdmoe_check_launch(what);
}

int hdmoe_launch_quant_rows(const void* x_bf16, int64_t rows, int D, const float* scale_input_dev,
                            const float* scale_input_also_dev, void* out_fp8, hipStream_t s, const char* what) {
  hipLaunchKernelGGL(quant_rows_kernel, dim3(row_blocks(rows)), dim3(THREADS), 0, s, static_cast<const uint4*>(x_bf16),
                     (long)rows, D / 8, scale_input_dev, scale_input_also_dev, static_cast<uint2*>(out_fp8));
  return hdmoe_check_launch(what);
}

extern "C" int hdmoe_quant_fp8(const void* x_bf16, int64_t rows, int D, const float* scale_input_dev, void* out_fp8,
                               hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(out_fp8);
  if (rows < 0 || D <= 0 || D % 8 != 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_quant_fp8: rows=%lld D=%d (D must be a positive multiple of 8)",
                      (long long)rows, D);
  if (rows == 0) return HDMOE_OK;
  return hdmoe_launch_quant_rows(x_bf16, rows, D, scale_input_dev, scale_input_dev, out_fp8,
                                 static_cast<hipStream_t>(stream), "hdmoe_quant_fp8");
}

extern "C" int hdmoe_quant_permute_fp8(const void* x_bf16, const int32_t* perm, const int32_t* offsets, int T, int D,
                                       int E, const float* const* scale_input, void* a_fp8, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(perm);
  HDMOE_REQUIRE_PTR(offsets);
  HDMOE_REQUIRE_PTR(scale_input);
  HDMOE_REQUIRE_PTR(a_fp8);
  if (T < 0 || D <= 0 || D % 8 != 0 || E < 1 || E > HDMOE_MAX_EXPERTS)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_quant_permute_fp8: T=%d D=%d E=%d", T, D, E);
  if (T == 0) return HDMOE_OK;
  ScalePtrs sp;
  for (int e = 0; e < HDMOE_MAX_EXPERTS; ++e) sp.p[e] = e < E ? scale_input[e] : nullptr;
  return hdmoe_launch_quant_dispatch(x_bf16, perm, offsets, T, D, E, scale_input, nullptr, false, a_fp8,
                                     static_cast<hipStream_t>(stream), "hdmoe_quant_permute_fp8");
}

extern "C" int hdmoe_permute_bf16(const void* x_bf16, const int32_t* perm, int T, int D, void* a_bf16,
                                  hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(perm);
  HDMOE_REQUIRE_PTR(a_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_permute_bf16: T=%d D=%d", T, D);
  if (T == 0) return HDMOE_OK;
  const int rows = T * HDMOE_TOPK;
  hipLaunchKernelGGL(permute_rows_kernel, dim3(row_blocks(rows)), dim3(THREADS), 0,
                     static_cast<hipStream_t>(stream), static_cast<const uint4*>(x_bf16), perm, rows, D / 8,
                     static_cast<uint4*>(a_bf16));
  return hdmoe_check_launch("hdmoe_permute_bf16");
}

extern "C" int hdmoe_silu_mul_bf16(const void* a_bf16, const void* b_bf16, int64_t n, void* out_bf16,
                                   hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(a_bf16);
  HDMOE_REQUIRE_PTR(b_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (n < 0 || n % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_silu_mul_bf16: n=%lld must be a multiple of 8", (long long)n);
  if (n == 0) return HDMOE_OK;
  const long n16 = n / 8;
  long blocks = (n16 + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 16) blocks = HDMOE_NUM_CU * 16;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((int)blocks), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(a_bf16), static_cast<const uint4*>(b_bf16), n16,
                     static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch("hdmoe_silu_mul_bf16");
}

extern "C" int hdmoe_gelu_bf16(const void* x_bf16, int64_t n, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (n < 0 || n % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_gelu_bf16: n=%lld must be a multiple of 8", (long long)n);
  if (n == 0) return HDMOE_OK;
  const int64_t n8 = n / 8;
  int64_t blocks = (n8 + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 8) blocks = HDMOE_NUM_CU * 8;
  hipLaunchKernelGGL(gelu_kernel<HdmoeBf16>, dim3((unsigned)blocks), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(x_bf16), n8, static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch("hdmoe_gelu_bf16");
}

extern "C" int hdmoe_gelu_f16(const void* x_f16, int64_t n, void* out_f16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_f16);
  HDMOE_REQUIRE_PTR(out_f16);
  if (n < 0 || n % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_gelu_f16: n=%lld must be a multiple of 8", (long long)n);
  if (n == 0) return HDMOE_OK;
  const int64_t n8 = n / 8;
  int64_t blocks = (n8 + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 8) blocks = HDMOE_NUM_CU * 8;
  hipLaunchKernelGGL(gelu_kernel<HdmoeF16>, dim3((unsigned)blocks), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(x_f16), n8, static_cast<uint4*>(out_f16));
  return hdmoe_check_launch("hdmoe_gelu_f16");
}

extern "C" int hdmoe_renorm_top2_bf16(const void* topk_weight_bf16, int T, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(topk_weight_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (T < 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_renorm_top2_bf16: T=%d", T);
  if (T == 0) return HDMOE_OK;
  int blocks = (T + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 4) blocks = HDMOE_NUM_CU * 4;
  hipLaunchKernelGGL(renorm_top2_kernel, dim3(blocks), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint32_t*>(topk_weight_bf16), T, static_cast<uint32_t*>(out_bf16));
  return hdmoe_check_launch("hdmoe_renorm_top2_bf16");
}

// The combine of a layer over the fp32 partial sums of a down projection cut along K (combine_partials_kernel).
// experts[e].scale_w2 / scale_in2 and the shared expert's are the scales of the rows (fp8 weights only).
int hdmoe_launch_combine_partials(const float* partial, long long part_stride, const HdmoeSplitPlan& plan,
                                  int rows_dyn, int n_dyn,
                                  const int32_t* offsets, bool fp8, const hdmoe_ffn_weights* experts,
                                  const hdmoe_ffn_weights* shared, const int32_t* inv_perm, const void* topk_weight_bf16,
                                  const void* gate_bf16, const void* residual_bf16, int tokens_per_batch, int T, int D,
                                  void* out_bf16, hipStream_t s, const char* what) {
  if (n_dyn < 0 || n_dyn > HDMOE_MAX_EXPERTS) return hdmoe_fail(HDMOE_E_SHAPE, "%s: %d experts", what, n_dyn);
  CombinePartialArgs pa;
  memset(&pa, 0, sizeof(pa));
  pa.partial = partial;
  pa.part_stride = part_stride;
  if (plan.n < 1 || plan.n > HDMOE_PLAN_MAX) return hdmoe_fail(HDMOE_E_SHAPE, "%s: split plan with %d entries", what, plan.n);
  pa.plan = plan;
  pa.rows_dyn = rows_dyn;
  pa.n_dyn = n_dyn;
  pa.fp8 = fp8 ? 1 : 0;
  pa.has_shared = shared != nullptr ? 1 : 0;
  pa.offsets = offsets;
  for (int e = 0; e < n_dyn; ++e) { pa.sw[e] = experts[e].scale_w2; pa.sin[e] = experts[e].scale_in2; }
  if (shared != nullptr) { pa.sw[n_dyn] = shared->scale_w2; pa.sin[n_dyn] = shared->scale_in2; }
  CombineExtra ex;
  ex.gate = static_cast<const uint4*>(gate_bf16);
  ex.residual = static_cast<const uint4*>(residual_bf16);
  ex.tokens_per_batch = tokens_per_batch > 0 ? tokens_per_batch : 1;
  const int row16 = D / 8;
  const long units = (long)T * ((row16 + 63) / 64);
  hipLaunchKernelGGL(combine_partials_kernel<HdmoeBf16>, dim3(row_blocks(units)), dim3(THREADS), 0, s, pa,
                     reinterpret_cast<const int2*>(inv_perm), static_cast<const uint32_t*>(topk_weight_bf16), T, row16, ex,
                     static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch(what);
}

int hdmoe_launch_combine(const void* y_sorted_bf16, const int32_t* inv_perm, const void* topk_weight_bf16,
                         const void* shared_bf16, const void* gate_bf16, const void* residual_bf16, int tokens_per_batch,
                         int T, int D, void* out_bf16, hipStream_t s, const char* what, bool f16 = false) {
  CombineExtra ex;
  ex.gate = static_cast<const uint4*>(gate_bf16);
  ex.residual = static_cast<const uint4*>(residual_bf16);
  ex.tokens_per_batch = tokens_per_batch > 0 ? tokens_per_batch : 1;
  if (f16)
    hipLaunchKernelGGL(combine_kernel<HdmoeF16>, dim3(row_blocks(T)), dim3(THREADS), 0, s,
                       static_cast<const uint4*>(y_sorted_bf16), reinterpret_cast<const int2*>(inv_perm),
                       static_cast<const uint32_t*>(topk_weight_bf16), static_cast<const uint4*>(shared_bf16), T, D / 8,
                       ex, static_cast<uint4*>(out_bf16));
  else
    hipLaunchKernelGGL(combine_kernel<HdmoeBf16>, dim3(row_blocks(T)), dim3(THREADS), 0, s,
                       static_cast<const uint4*>(y_sorted_bf16), reinterpret_cast<const int2*>(inv_perm),
                       static_cast<const uint32_t*>(topk_weight_bf16), static_cast<const uint4*>(shared_bf16), T, D / 8,
                       ex, static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch(what);
}

extern "C" int hdmoe_combine_f16(const void* y_sorted_f16, const int32_t* inv_perm, const void* topk_weight_f16,
                                 const void* shared_f16, int T, int D, void* out_f16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(y_sorted_f16);
  HDMOE_REQUIRE_PTR(inv_perm);
  HDMOE_REQUIRE_PTR(topk_weight_f16);
  HDMOE_REQUIRE_PTR(out_f16);
  if (T < 0 || D <= 0 || D % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_combine_f16: T=%d D=%d", T, D);
  if (T == 0) return HDMOE_OK;
  return hdmoe_launch_combine(y_sorted_f16, inv_perm, topk_weight_f16, shared_f16, nullptr, nullptr, 1, T, D, out_f16,
                              static_cast<hipStream_t>(stream), "hdmoe_combine_f16", true);
}

extern "C" int hdmoe_combine(const void* y_sorted_bf16, const int32_t* inv_perm, const void* topk_weight_bf16,
                             const void* shared_bf16, int T, int D, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(y_sorted_bf16);
  HDMOE_REQUIRE_PTR(inv_perm);
  HDMOE_REQUIRE_PTR(topk_weight_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_combine: T=%d D=%d", T, D);
  if (T == 0) return HDMOE_OK;
  return hdmoe_launch_combine(y_sorted_bf16, inv_perm, topk_weight_bf16, shared_bf16, nullptr, nullptr, 1, T, D, out_bf16,
                              static_cast<hipStream_t>(stream), "hdmoe_combine");
}

extern "C" int hdmoe_combine_gated_residual(const void* y_sorted_bf16, const int32_t* inv_perm,
                                            const void* topk_weight_bf16, const void* shared_bf16,
                                            const void* gate_bf16, const void* residual_bf16, int tokens_per_batch,
                                            int T, int D, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(y_sorted_bf16);
  HDMOE_REQUIRE_PTR(inv_perm);
  HDMOE_REQUIRE_PTR(topk_weight_bf16);
  HDMOE_REQUIRE_PTR(gate_bf16);
  HDMOE_REQUIRE_PTR(residual_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0 || tokens_per_batch <= 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_combine_gated_residual: T=%d D=%d tokens_per_batch=%d", T, D, tokens_per_batch);
  if (T == 0) return HDMOE_OK;
  return hdmoe_launch_combine(y_sorted_bf16, inv_perm, topk_weight_bf16, shared_bf16, gate_bf16, residual_bf16,
                              tokens_per_batch, T, D, out_bf16, static_cast<hipStream_t>(stream),
                              "hdmoe_combine_gated_residual");
}

extern "C" int hdmoe_gated_residual_bf16(const void* y_bf16, const void* gate_bf16, const void* residual_bf16,
                                         int tokens_per_batch, int T, int D, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(y_bf16);
  HDMOE_REQUIRE_PTR(gate_bf16);
  HDMOE_REQUIRE_PTR(residual_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0 || tokens_per_batch <= 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_gated_residual_bf16: T=%d D=%d tokens_per_batch=%d", T, D, tokens_per_batch);
  if (T == 0) return HDMOE_OK;
  hipLaunchKernelGGL(gated_residual_kernel, dim3(row_blocks(T)), dim3(THREADS), 0, static_cast<hipStream_t>(stream),
                     static_cast<const uint4*>(y_bf16), static_cast<const uint4*>(gate_bf16),
                     static_cast<const uint4*>(residual_bf16), T, D / 8, tokens_per_batch, static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch("hdmoe_gated_residual_bf16");
}

extern "C" int hdmoe_scale_to_bf16(int src_dtype, const void* src, int64_t n, const float* scale_dev, void* out_bf16,
                                   hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(src);
  HDMOE_REQUIRE_PTR(scale_dev);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (n < 0 || n % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_scale_to_bf16: n=%lld must be a multiple of 8", (long long)n);
  if (src_dtype != HDMOE_W_BF16 && src_dtype != HDMOE_W_E4M3FN)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_scale_to_bf16: src_dtype=%d", src_dtype);
  if (n == 0) return HDMOE_OK;
  const long n8 = n / 8;
  long blocks = (n8 + THREADS - 1) / THREADS;
  if (blocks > HDMOE_NUM_CU * 16) blocks = HDMOE_NUM_CU * 16;
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (src_dtype == HDMOE_W_E4M3FN)
    hipLaunchKernelGGL(scale_fp8_to_bf16_kernel, dim3((int)blocks), dim3(THREADS), 0, s, static_cast<const uint2*>(src), n8,
                       scale_dev, static_cast<uint4*>(out_bf16));
  else
    hipLaunchKernelGGL(scale_bf16_kernel, dim3((int)blocks), dim3(THREADS), 0, s, static_cast<const uint4*>(src), n8,
                       scale_dev, static_cast<uint4*>(out_bf16));
  return hdmoe_check_launch("hdmoe_scale_to_bf16");
}
