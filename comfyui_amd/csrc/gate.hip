// Gate kernels: logits = x . Wg^T, softmax, top-2 with lowest-index tie-break.
// Replaces MoEGate.forward (/root/reference/comfy/ldm/hidream/model.py:263-283).
//
// One token per wavefront. Lane l owns the 8-element groups starting at element
// l*8 + c*512 (c = 0, 1, ...): a 16-byte load per lane and chunk, so a wave reads
// 1 KiB of the token row per load instruction, fully coalesced. A lane needs the
// same slice of Wg for every token: the kernels for HiDream's shape keep Wg in LDS
// as fp32, the generic kernel re-reads it through the caches for four tokens at a
// time. The E dot products are accumulated in fp32 with fma in ascending element
// order per lane and reduced across the wave with an xor butterfly (32, 16, 8, 4,
// 2, 1). That order is fixed on purpose: it is the order the CPU checker restates,
// which makes logits, scores and therefore the routing reproducible bit for bit.
//
// HBM traffic per token: D*2 bytes read, 12 bytes written (plus D bytes where the
// kernel also casts the token to fp8 for the expert GEMMs).
#include "common.h"
#include "numfmt.h"
#include "quant.h"

#pragma clang fp contract(off)

namespace {

constexpr int WAVES_PER_BLOCK = 4;
constexpr int GENERIC_TOKENS_PER_TRIP = 4;   // tokens a wave of the generic kernel takes together

__device__ __forceinline__ float exp_neg(float x) {
  // exp(x), x <= 0: ln2 split range reduction, degree-5 polynomial, exponent
  // added through the bit pattern. Only fp32 fma/mul/add, so results do not
  // depend on a math library.
  x = x < -80.0f ? -80.0f : x;
  float n = __builtin_rintf(x * 1.44269504088896341f);
  float r = __builtin_fmaf(n, -0.693359375f, x);
  r = __builtin_fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = __builtin_fmaf(p, r, 1.3981999507e-3f);
  p = __builtin_fmaf(p, r, 8.3334519073e-3f);
  p = __builtin_fmaf(p, r, 4.1665795894e-2f);
  p = __builtin_fmaf(p, r, 1.6666665459e-1f);
  p = __builtin_fmaf(p, r, 5.0000001201e-1f);
  float z = r * r;
  float y = __builtin_fmaf(p, z, r);
  y = y + 1.0f;
  return __uint_as_float(__float_as_uint(y) + ((uint32_t)(int32_t)n << 23));
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// The element format of x, the gate weight and the routing weights: bf16 (HiDream, Hunyuan3D) or fp16 (the dtype
// Hunyuan3D runs in where the device takes it). Logits and scores are rounded to that format between the steps.
struct GateBf16 {
  static __device__ __forceinline__ float lo(uint32_t u) { return bf16_lo(u); }
  static __device__ __forceinline__ float hi(uint32_t u) { return bf16_hi(u); }
  static __device__ __forceinline__ float round(float f) { return hdmoe_round_bf16(f); }
  static __device__ __forceinline__ uint32_t pack(float a, float b) {
    return (uint32_t)hdmoe_f32_to_bf16(a) | ((uint32_t)hdmoe_f32_to_bf16(b) << 16);
  }
};
typedef HdmoeF16 GateF16;

template <class A = GateBf16>
__device__ __forceinline__ float dot8(const uint4& a, const uint4& b, float acc) {
  acc = __builtin_fmaf(A::lo(a.x), A::lo(b.x), acc);
  acc = __builtin_fmaf(A::hi(a.x), A::hi(b.x), acc);
  acc = __builtin_fmaf(A::lo(a.y), A::lo(b.y), acc);
  acc = __builtin_fmaf(A::hi(a.y), A::hi(b.y), acc);
  acc = __builtin_fmaf(A::lo(a.z), A::lo(b.z), acc);
  acc = __builtin_fmaf(A::hi(a.z), A::hi(b.z), acc);
  acc = __builtin_fmaf(A::lo(a.w), A::lo(b.w), acc);
  acc = __builtin_fmaf(A::hi(a.w), A::hi(b.w), acc);
  return acc;
}

// Sum over the wave in the fixed butterfly order v[l] + v[l ^ off], off = 32, 16, 8, 4, 2, 1, every lane ending
// with the total. No LDS traffic: the halves and the 16-lane rows are exchanged with the lane-swap instructions,
// the rest with DPP. After the first two steps the values repeat every 16 lanes, so the rotate by 8 inside a row
// is the xor-8 partner, and once they repeat every 8 lanes the rotate by 4 is the xor-4 partner; fp32 addition is
// commutative, so each lane forms exactly the sum the plain xor shuffle would.
__device__ __forceinline__ float wave_sum(float v) {
  uint32_t b = __float_as_uint(v);
  auto h = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  v = __uint_as_float(h[0]) + __uint_as_float(h[1]);
  b = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane16_swap(b, b, false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  int x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x128, 0xf, 0xf, false));  // row_ror:8
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x124, 0xf, 0xf, false));  // row_ror:4
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x4e, 0xf, 0xf, false));   // quad_perm:[2,3,0,1]
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0xb1, 0xf, 0xf, false));   // quad_perm:[1,0,3,2]
  return v;
}

template <int E, class A = GateBf16>
__device__ __forceinline__ void finish_token(float (&logit)[E], int lane, int t, int32_t* idx,
                                             uint16_t* wout, int& first, int& second) {
#pragma unroll
  for (int e = 0; e < E; ++e) {
    logit[e] = A::round(wave_sum(logit[e]));  // F.linear output is a tensor of the activation format
  }
  float mx = logit[0];
#pragma unroll
  for (int e = 1; e < E; ++e) mx = logit[e] > mx ? logit[e] : mx;
  float ex[E];
  float sum = 0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    ex[e] = exp_neg(logit[e] - mx);
    sum = sum + ex[e];
  }
  float score[E];
#pragma unroll
  for (int e = 0; e < E; ++e) score[e] = A::round(__fdiv_rn(ex[e], sum));  // so is the softmax output
  // first two of a stable descending sort: strict '>' keeps the lower index on ties
  int i0 = 0;
  float s0 = score[0];
#pragma unroll
  for (int e = 1; e < E; ++e)
    if (score[e] > s0) { s0 = score[e]; i0 = e; }
  int i1 = -1;
  float s1 = 0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    if (e == i0) continue;
    if (i1 < 0 || score[e] > s1) { s1 = score[e]; i1 = e; }
  }
  first = i0;
  second = i1;
  if (lane == 0) {
    reinterpret_cast<int2*>(idx)[t] = make_int2(i0, i1);
    reinterpret_cast<uint32_t*>(wout)[t] = A::pack(s0, s1);
  }
}

__device__ __forceinline__ void unpack8(const uint4& a, float (&f)[8]) {
  f[0] = bf16_lo(a.x); f[1] = bf16_hi(a.x); f[2] = bf16_lo(a.y); f[3] = bf16_hi(a.y);
  f[4] = bf16_lo(a.z); f[5] = bf16_hi(a.z); f[6] = bf16_lo(a.w); f[7] = bf16_hi(a.w);
}

__device__ __forceinline__ void round2(float& a, float& b) {
  const uint32_t p = hdmoe_dev_pack_bf16(a, b);
  a = __uint_as_float(p << 16);
  b = __uint_as_float(p & 0xffff0000u);
}

__device__ __forceinline__ uint4 modulate8(const uint4& xv, const uint4& sc, const uint4& sh, float mean, float rstd) {
  float x[8], a[8], b[8];
  unpack8(xv, x);
  unpack8(sc, a);
  unpack8(sh, b);
  uint32_t o[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    // two elements at a time: one packed conversion (v_cvt_pk_bf16_f32, round to nearest even) per rounding point
    float n0 = (x[2 * j] - mean) * rstd, n1 = (x[2 * j + 1] - mean) * rstd;  // LayerNorm output as a bf16 tensor
    round2(n0, n1);
    float m0 = 1.0f + a[2 * j], m1 = 1.0f + a[2 * j + 1];                    // (1 + scale)
    round2(m0, m1);
    float p0 = n0 * m0, p1 = n1 * m1;                                        // n * (1 + scale)
    round2(p0, p1);
    o[j] = hdmoe_dev_pack_bf16(p0 + b[2 * j], p1 + b[2 * j + 1]);            // + shift
  }
  return make_uint4(o[0], o[1], o[2], o[3]);
}

// LayerNorm statistics of a row held in registers (NCHUNK x 8 elements per lane): the two passes and the fixed
// fp32 order documented at the LayerNorm kernel below.
template <int NCHUNK>
__device__ __forceinline__ void ln_stats(const uint4 (&v)[NCHUNK], float fD, float eps, float& mean, float& rstd) {
  float s = 0.0f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float f[8];
    unpack8(v[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) s = s + f[j];
  }
  mean = __fdiv_rn(wave_sum(s), fD);
  float s2 = 0.0f;
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float f[8];
    unpack8(v[c], f);
#pragma unroll
    for (int j = 0; j < 8; ++j) { const float d = f[j] - mean; s2 = __builtin_fmaf(d, d, s2); }
  }
  rstd = __fdiv_rn(1.0f, __builtin_sqrtf(__fdiv_rn(wave_sum(s2), fD) + eps));
}

// D == NCHUNK * 512: the lane's Wg slice lives in registers.
// Optional second output of both kernels (QUANT): the token's fp8 rows for the expert GEMMs, cast while the row
// is at hand. Row 2t+s of xq_routed (NULL: every Linear that reads the tokens shares one scale_input, the shared copy
// serves them all) is x[t] cast with the scale_input of the expert in slot s, row t of xq_shared
// the cast for the shared expert; the GEMM reads them through the dispatch permutation.
struct GateQuant {
  HdmoeScalePtrs scale_in;    // per expert, NULL = clamp rule
  const float* shared_scale;
  uint2* xq_routed;           // [2T, D] e4m3fn
  uint2* xq_shared;           // [T, D] e4m3fn or NULL
  // Decisions and checks that depend on the VALUES behind the scale pointers are made here, on the device, from
  // those values: the host would have to read them back to know them, and a copy it keeps goes stale when a scale
  // tensor is written in place.
  //   decide != 0: both outputs are given and the kernel chooses. If every expert (and the shared expert) casts the
  //     tokens with the same factor, it writes one row per token to xq_shared and 1 to *layout_flag; else the rows
  //     2t, 2t+1 of xq_routed (and the shared expert's copy if with_shared) and 0 to *layout_flag. The GEMM that
  //     follows reads the flag and the matching operand.
  //   scale_in3 / shared_scale3: scale_input of the w3 Linears. w1 and w3 read one cast of the tokens, made with
  //     w1's factor; where w3's factor differs the cast cannot serve both, the rows are written as NaN (so is then
  //     the layer's output) and *scale_check, if given, is set to 1.
  int decide, with_shared;
  int32_t* layout_flag;
  int32_t* scale_check;
  HdmoeScalePtrs scale_in3;
  const float* shared_scale3;
  // LN variant of the register kernel: the row is LayerNorm(x) * (1 + scale[b]) + shift[b] (as ln_modulate_kernel
  // computes it, bit for bit), b = token / tokens_per_batch; the normalised tokens are never written as bf16
  const uint4* mod_scale;     // [batch, D] bf16
  const uint4* mod_shift;
  int tokens_per_batch;
  float ln_eps;
};

// Token -> wave mapping of both kernels, one of two:
//   tpb > 0: block b owns tokens [b * tpb, (b + 1) * tpb), its waves take them in turn (wave w: b * tpb + w,
//     + WAVES_PER_BLOCK, ...). A block then knows the expert histogram of a contiguous token range, which is the
//     first pass of the dispatch's counting sort: block b writes its E counts to block_hist[b * E ..] and the
//     dispatch needs no counting launch of its own;
//   tpb == 0: the waves of the grid stride over the tokens (wave g: g, g + waves in the grid, ...), so that at any
//     moment the grid reads one contiguous stretch of x; no histograms (the stage entry points).
struct TokenWalk { int first, end, step; };
__device__ __forceinline__ TokenWalk token_walk(int T, int tpb) {
  const int wv = threadIdx.x >> 6;
  if (tpb > 0) return {(int)blockIdx.x * tpb + wv, min(T, (int)(blockIdx.x + 1) * tpb), WAVES_PER_BLOCK};
  return {(int)blockIdx.x * WAVES_PER_BLOCK + wv, T, (int)gridDim.x * WAVES_PER_BLOCK};
}

template <int E, int NWAVES = WAVES_PER_BLOCK>
__device__ __forceinline__ void write_block_hist(const int (&cnt)[E], int32_t* __restrict__ block_hist) {
  __shared__ int32_t wave_cnt[NWAVES][E];
  if (block_hist == nullptr) return;  // kernel argument: the same for every thread
  const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  if (lane == 0) {
#pragma unroll
    for (int e = 0; e < E; ++e) wave_cnt[wv][e] = cnt[e];
  }
  __syncthreads();
  if (threadIdx.x < E) {
    int32_t sum = 0;
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) sum += wave_cnt[w][threadIdx.x];
    block_hist[(size_t)blockIdx.x * E + threadIdx.x] = sum;
  }
}

// ---- the kernels for D = NCHUNK * 512 and up to 4 experts -----------------------------------------------------
// One token per wave and trip, sixteen waves per CU. The gate weight sits in LDS as fp32 (E * D * 4 bytes: 40 KiB
// for HiDream), written once per block, so that the dot products are fused multiply-adds on LDS operands with
// nothing to unpack but the token. The E partial sums per lane are added up across the wave in the butterfly order
// of wave_sum, but folded: at the step with offset 32 the lower half of the wave keeps the sums of one expert and
// the upper half those of another (v[l] + v[l ^ 32] is the same number in both lanes, so computing it once loses
// nothing), at offset 16 the four 16-lane rows end up with the four experts, and the last four steps run on one
// register instead of four. Row e of that register then holds logit e; softmax is evaluated once on the rows (its
// exponential and division once per token instead of once per expert), the E scores come back through lane reads,
// and the top-2 selection and everything after it is wave-uniform.
// Every floating-point operation has the operands and the order of the plain one-token form (dot8, wave_sum,
// finish_token), so the results are the same bit for bit.
__device__ __forceinline__ float fold32(float a, float b) {
  auto h = __builtin_amdgcn_permlane32_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(h[0]) + __uint_as_float(h[1]);   // lanes 0-31: a[l] + a[l + 32]; lanes 32-63: the same for b
}
__device__ __forceinline__ float fold16(float a, float b) {
  auto h = __builtin_amdgcn_permlane16_swap(__float_as_uint(a), __float_as_uint(b), false, false);
  return __uint_as_float(h[0]) + __uint_as_float(h[1]);   // rows 0, 2: a's rows 0 + 1, 2 + 3; rows 1, 3: b's
}
__device__ __forceinline__ float row_sum(float v) {      // offsets 8, 4, 2, 1 inside every 16-lane row
  int x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x128, 0xf, 0xf, false));  // row_ror:8
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x124, 0xf, 0xf, false));  // row_ror:4
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0x4e, 0xf, 0xf, false));   // quad_perm:[2,3,0,1]
  x = __float_as_int(v);
  v = v + __int_as_float(__builtin_amdgcn_update_dpp(x, x, 0xb1, 0xf, 0xf, false));   // quad_perm:[1,0,3,2]
  return v;
}
__device__ __forceinline__ float lane_value(float v, int lane) {
  return __uint_as_float(__builtin_amdgcn_readlane(__float_as_uint(v), lane));
}
// partial sums of up to 4 experts -> one register whose 16-lane row e holds the wave total of expert e
template <int E>
__device__ __forceinline__ float expert_rows(const float (&acc)[E]) {
  const float a0 = acc[0], a1 = acc[1], a2 = E > 2 ? acc[2] : 0.0f, a3 = E > 3 ? acc[3] : 0.0f;
  return row_sum(fold16(fold32(a0, a2), fold32(a1, a3)));
}

// logits in rows -> routing of one token (wave-uniform): indices, the two scores
template <int E>
__device__ __forceinline__ void finish_rows(float rows, int& i0, int& i1, float& s0, float& s1) {
  const float lg = GateBf16::round(rows);          // F.linear output is a bf16 tensor
  float l[E];
#pragma unroll
  for (int e = 0; e < E; ++e) l[e] = lane_value(lg, 16 * e);
  float mx = l[0];
#pragma unroll
  for (int e = 1; e < E; ++e) mx = l[e] > mx ? l[e] : mx;
  const float ex = exp_neg(lg - mx);               // row e: exp(logit e - max); rows past E hold nothing of use
  float sum = 0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) sum = sum + lane_value(ex, 16 * e);
  const float sc = GateBf16::round(__fdiv_rn(ex, sum));   // so is the softmax output
  float score[E];
#pragma unroll
  for (int e = 0; e < E; ++e) score[e] = lane_value(sc, 16 * e);
  // first two of a stable descending sort: strict '>' keeps the lower index on ties
  i0 = 0;
  s0 = score[0];
#pragma unroll
  for (int e = 1; e < E; ++e)
    if (score[e] > s0) { s0 = score[e]; i0 = e; }
  i1 = -1;
  s1 = 0.0f;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    if (e == i0) continue;
    if (i1 < 0 || score[e] > s1) { s1 = score[e]; i1 = e; }
  }
}

// E dot products of one token row with the fp32 gate weight in LDS. Unit (e, c, lane) of the bf16 weight (8
// elements) is the two float4 at [(e * NCHUNK + c) * 2 + half][lane]: a lane's reads are 16 bytes wide and
// lane-contiguous (no bank conflicts). Step s = c * E + e multiplies chunk c with the unit of expert e. The LDS reads
// run RA steps ahead of the arithmetic and no further: each step's empty statement defines the lane offset the next
// reads use and consumes the sum of the step before, so the compiler can neither gather all reads at the top (the
// whole slice, E * D / 64 values, in registers: that is what it does when left alone, and it costs the occupancy
// these kernels live on) nor hoist them out of the token loop.
template <int E, int NCHUNK, int RA>
__device__ __forceinline__ void dot_rows(const uint4 (&row)[NCHUNK], const float4* wf, int lane, float (&acc)[E]) {
  constexpr int STEPS = NCHUNK * E;
#pragma unroll
  for (int e = 0; e < E; ++e) acc[e] = 0.0f;
  int wlane = lane;
  asm volatile("" : "+v"(wlane));
  float4 wlo[RA], whi[RA];
#pragma unroll
  for (int s = 0; s < RA && s < STEPS; ++s) {
    const int u = (s % E) * NCHUNK + s / E;
    wlo[s] = wf[(u * 2 + 0) * 64 + wlane];
    whi[s] = wf[(u * 2 + 1) * 64 + wlane];
  }
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    float xa[8];
    unpack8(row[c], xa);
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const int st = c * E + e;
      const float4 lo = wlo[st % RA], hi = whi[st % RA];
      if (st + RA < STEPS) {
        const int u = ((st + RA) % E) * NCHUNK + (st + RA) / E;
        asm volatile("" : "+v"(wlane), "+v"(acc[e == 0 ? E - 1 : e - 1]));
        wlo[st % RA] = wf[(u * 2 + 0) * 64 + wlane];
        whi[st % RA] = wf[(u * 2 + 1) * 64 + wlane];
      }
      const float w8[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
      for (int j = 0; j < 8; ++j) acc[e] = __builtin_fmaf(xa[j], w8[j], acc[e]);
    }
  }
}

// What the cast needs to know about the scale values (see GateQuant), the same in every wave of the grid.
template <int E>
struct CastFacts {
  float inv_e[E], invs;        // (1 / scale_input).to(bf16) per expert and for the shared expert; NaN where w1 and
                               // w3 of a feed-forward disagree: every product and so every byte written is NaN
  bool one_row, with_shared;   // one row per token for all readers; per-slot rows plus the shared expert's copy
};
// The raw values are asked for early (before the weight fill's barrier), the facts derived behind it.
template <int E>
struct ScaleValues { float in1[E], in3[E], shared1, shared3; };
template <int E>
__device__ __forceinline__ ScaleValues<E> request_scales(const GateQuant& q) {
  ScaleValues<E> v;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    v.in1[e] = q.scale_in.p[e] != nullptr ? *q.scale_in.p[e] : 0.0f;
    v.in3[e] = q.scale_in3.p[e] != nullptr ? *q.scale_in3.p[e] : 0.0f;
  }
  v.shared1 = q.shared_scale != nullptr ? *q.shared_scale : 0.0f;
  v.shared3 = q.shared_scale3 != nullptr ? *q.shared_scale3 : 0.0f;
  return v;
}
template <int E>
__device__ __forceinline__ CastFacts<E> cast_facts(const GateQuant& q, const ScaleValues<E>& v) {
  // NULL pointer: the clamp rule's marker
  auto inv_of = [](const float* p, float s) { return p == nullptr ? -1.0f : hdmoe_dev_round_bf16(__fdiv_rn(1.0f, s)); };
  CastFacts<E> f;
  bool ok13 = true, same = true;
#pragma unroll
  for (int e = 0; e < E; ++e) {
    f.inv_e[e] = hdmoe_q_uniform(inv_of(q.scale_in.p[e], v.in1[e]));
    if (q.scale_in3.p[e] != q.scale_in.p[e]) ok13 = ok13 && inv_of(q.scale_in3.p[e], v.in3[e]) == f.inv_e[e];
  }
  f.invs = hdmoe_q_uniform(inv_of(q.shared_scale, v.shared1));
  if (q.shared_scale3 != q.shared_scale) ok13 = ok13 && inv_of(q.shared_scale3, v.shared3) == f.invs;
#pragma unroll
  for (int e = 0; e < E; ++e) same = same && f.inv_e[e] == f.invs;
  f.one_row = q.decide ? same : q.xq_routed == nullptr;
  f.with_shared = q.decide ? q.with_shared != 0 : q.xq_shared != nullptr;
  if (!ok13) {
    f.invs = __builtin_nanf("");
#pragma unroll
    for (int e = 0; e < E; ++e) f.inv_e[e] = f.invs;
  }
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (q.decide) *q.layout_flag = same ? 1 : 0;
    if (!ok13 && q.scale_check != nullptr) *q.scale_check = 1;
  }
  return f;
}

// the fp8 rows of token t: one row for all readers, or a row per slot (and the shared expert's copy)
template <int E, int NCHUNK>
__device__ __forceinline__ void cast_token(const uint4 (&row)[NCHUNK], int t, int i0, int i1, const CastFacts<E>& f,
                                           const GateQuant& q, int lane) {
  constexpr int ROW16 = NCHUNK * 64;
  if (f.one_row) {
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) q.xq_shared[(size_t)t * ROW16 + c * 64 + lane] = hdmoe_q_8(row[c], f.invs);
    return;
  }
  float inv0 = f.inv_e[0], inv1 = f.inv_e[0];
#pragma unroll
  for (int e = 1; e < E; ++e) {
    inv0 = i0 == e ? f.inv_e[e] : inv0;
    inv1 = i1 == e ? f.inv_e[e] : inv1;
  }
  inv0 = hdmoe_q_uniform(inv0);
  inv1 = hdmoe_q_uniform(inv1);
  uint2* r0 = q.xq_routed + (size_t)(2 * t) * ROW16;
  const bool same01 = inv0 == inv1, same0s = inv0 == f.invs;  // equal scales: cast once, store again
#pragma unroll
  for (int c = 0; c < NCHUNK; ++c) {
    const uint2 v0 = hdmoe_q_8(row[c], inv0);
    r0[c * 64 + lane] = v0;
    r0[ROW16 + c * 64 + lane] = same01 ? v0 : hdmoe_q_8(row[c], inv1);
    if (f.with_shared) q.xq_shared[(size_t)t * ROW16 + c * 64 + lane] = same0s ? v0 : hdmoe_q_8(row[c], f.invs);
  }
}

// Three forms of one kernel, eight waves per block and two blocks per CU in each:
//   GATE_ROUTE  routing only (bf16 experts, the stage entry point): eight routing waves.
//   GATE_SPLIT  routing and the fp8 cast by different waves. Waves 0-3 route; their only stores are the 12 bytes of
//     routing per token. Waves 4-7 cast: they load the same tokens, cast them and store the fp8 rows, two rows in
//     flight, never touch the gate weight and pass the fill barrier at once. A wave that does both computes, then
//     casts and stores, and while its stores and next loads queue up behind those of every other wave its arithmetic
//     cannot issue (instructions issue in order); with two kinds of wave the arithmetic of one overlaps the memory
//     traffic of the other. The second read of a row comes from cache: both waves of a token sit on one CU and ask
//     for it at about the same time. The split needs a cast that does not depend on the routing, i.e. one cast
//     factor for every expert; where the scale values say otherwise (decided here, on the device) the cast waves
//     wait, and behind a barrier all eight waves write the per-slot rows from the routing the first four have left
//     in idx. Measured inside the layer (kernel start to last store, 8192 / 4096 / 256 tokens): 19 / 12 / 7 us
//     against 24 / 18 / 11 us with eight waves per CU that each route and cast two tokens per trip.
//   GATE_LN     LayerNorm + modulation in front (the block branch's form): about 800 vector instructions per token,
//     bound by arithmetic, so every wave does all of it for its tokens and nothing is computed twice (with the split
//     both kinds of wave would normalise the row: 115 instead of 81 us at 32768 tokens).
enum GateForm { GATE_ROUTE = 0, GATE_SPLIT = 1, GATE_LN = 2 };
constexpr int ROW_WAVES = 8;           // waves per block of the register kernels
constexpr int ROW_BLOCKS_PER_CU = 2;

template <int E, int NCHUNK, int FORM>
__global__ __launch_bounds__(ROW_WAVES * 64, ROW_WAVES * ROW_BLOCKS_PER_CU / 4) void gate_row_kernel(
    const uint4* __restrict__ x, const uint4* __restrict__ wg, int T, int tpb, int32_t* __restrict__ idx,
    uint16_t* __restrict__ wout, int32_t* __restrict__ block_hist, GateQuant q) {
  constexpr bool CAST = FORM != GATE_ROUTE, SPLIT = FORM == GATE_SPLIT, LN = FORM == GATE_LN;
  constexpr int RW = SPLIT ? ROW_WAVES / 2 : ROW_WAVES;   // routing waves per block
  constexpr int RA = LN ? 2 : 3;                          // LDS read-ahead; a third step spills in the LN form
  constexpr int ROW16 = NCHUNK * 64;                      // 16-byte units per row
  const int lane = threadIdx.x & 63;
  const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int rw = wv % RW;
  const bool caster = SPLIT && wv >= RW;
  // the tokens of wave rw (of either kind): block ranges, or strided over the grid (see TokenWalk)
  int t0, t_end, step;
  if (tpb > 0) {
    t0 = (int)blockIdx.x * tpb + rw;
    t_end = min(T, (int)(blockIdx.x + 1) * tpb);
    step = RW;
  } else {
    t0 = (int)blockIdx.x * RW + rw;
    t_end = T;
    step = (int)gridDim.x * RW;
  }
  const int t_first = t0;
  uint4 row[NCHUNK], nxt[NCHUNK];
  auto load_row = [&](int t, uint4 (&r)[NCHUNK]) {
#pragma unroll
    for (int c = 0; c < NCHUNK; ++c) r[c] = x[(size_t)t * ROW16 + c * 64 + lane];
  };
  // gate weight -> LDS as fp32, by the routing waves, requested in front of their first row; the scale values are
  // asked for before the barrier too, so that all three latencies pass together
  __shared__ float4 wf[E * NCHUNK * 2 * 64];
  constexpr int FILL = (E * ROW16 + RW * 64 - 1) / (RW * 64);
  uint4 wpart[FILL];
  if (!caster) {
#pragma unroll
    for (int k = 0; k < FILL; ++k) {
      const int i = threadIdx.x + k * RW * 64;
      wpart[k] = i < E * ROW16 ? wg[i] : make_uint4(0, 0, 0, 0);
    }
  }
  if (t0 < t_end) load_row(t0, row);
  ScaleValues<E> scales;
  if constexpr (CAST) scales = request_scales<E>(q);
  if (!caster) {
#pragma unroll
    for (int k = 0; k < FILL; ++k) {
      const int i = threadIdx.x + k * RW * 64;
      if (i < E * ROW16) {
        const uint4 v = wpart[k];
        const int unit = i >> 6, l = i & 63;
        wf[(unit * 2 + 0) * 64 + l] = make_float4(bf16_lo(v.x), bf16_hi(v.x), bf16_lo(v.y), bf16_hi(v.y));
        wf[(unit * 2 + 1) * 64 + l] = make_float4(bf16_lo(v.z), bf16_hi(v.z), bf16_lo(v.w), bf16_hi(v.w));
      }
    }
  }
  __syncthreads();
  CastFacts<E> facts;
  if constexpr (CAST) facts = cast_facts<E>(q, scales);

  int cnt[E];
#pragma unroll
  for (int e = 0; e < E; ++e) cnt[e] = 0;
  if (!caster) {
    for (; t0 < t_end; t0 += step) {
      const int tn = t0 + step;
      if (tn < t_end) load_row(tn, nxt);   // the next token's row, a trip ahead
      if constexpr (LN) {
        float m, r;
        ln_stats<NCHUNK>(row, (float)(NCHUNK * 512), q.ln_eps, m, r);
        const size_t b0 = (size_t)(t0 / q.tokens_per_batch) * ROW16;
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c)
          row[c] = modulate8(row[c], q.mod_scale[b0 + c * 64 + lane], q.mod_shift[b0 + c * 64 + lane], m, r);
      }
      float acc[E];
      dot_rows<E, NCHUNK, RA>(row, wf, lane, acc);
      int i0, i1;
      float s0, s1;
      finish_rows<E>(expert_rows<E>(acc), i0, i1, s0, s1);
      if (lane == 0) {
        reinterpret_cast<int2*>(idx)[t0] = make_int2(i0, i1);
        reinterpret_cast<uint32_t*>(wout)[t0] = GateBf16::pack(s0, s1);
      }
#pragma unroll
      for (int e = 0; e < E; ++e) cnt[e] += (i0 == e) + (i1 == e);
      if constexpr (LN) cast_token<E, NCHUNK>(row, t0, i0, i1, facts, q, lane);
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) row[c] = nxt[c];
    }
  } else if (facts.one_row) {
    // two rows in flight: the cast itself is a few instructions, the wave's time is memory latency
    if (t0 + step < t_end) load_row(t0 + step, nxt);
    for (; t0 < t_end; t0 += 2 * step) {
      auto cast_row = [&](int t, uint4 (&r)[NCHUNK]) {
        if (t >= t_end) return;
        uint2 o[NCHUNK];
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) o[c] = hdmoe_q_8(r[c], facts.invs);
        if (t + 2 * step < t_end) load_row(t + 2 * step, r);
#pragma unroll
        for (int c = 0; c < NCHUNK; ++c) q.xq_shared[(size_t)t * ROW16 + c * 64 + lane] = o[c];
      };
      cast_row(t0, row);
      cast_row(t0 + step, nxt);
    }
  }
  if constexpr (SPLIT) {
    if (!facts.one_row) {
      // a cast per slot: all eight waves, from the routing the first four have written (the barrier makes a block's
      // own global stores visible to its waves)
      __syncthreads();
      for (int t = t_first + (wv / RW) * step; t < t_end; t += 2 * step) {
        load_row(t, row);
        const int2 r = reinterpret_cast<const int2*>(idx)[t];
        cast_token<E, NCHUNK>(row, t, __builtin_amdgcn_readfirstlane(r.x), __builtin_amdgcn_readfirstlane(r.y), facts,
                              q, lane);
      }
    }
  }
  write_block_hist<E, ROW_WAVES>(cnt, block_hist);
}

// Any D that is a multiple of 8: Wg is re-read through the cache hierarchy.
template <int E, bool QUANT, class A = GateBf16>
__global__ __launch_bounds__(WAVES_PER_BLOCK * 64) void gate_top2_generic_kernel(
    const uint4* __restrict__ x, const uint4* __restrict__ wg, int T, int D, int tpb, int32_t* __restrict__ idx,
    uint16_t* __restrict__ wout, int32_t* __restrict__ block_hist, GateQuant q) {
  const int lane = threadIdx.x & 63;
  const int row16 = D / 8;
  const TokenWalk walk = token_walk(T, tpb);
  const int t_end = walk.end;
  int cnt[E];
#pragma unroll
  for (int e = 0; e < E; ++e) cnt[e] = 0;
  // the decisions and checks on the scale values (see GateQuant), once per wave
  bool one_row = false, with_shared = false, ok13 = true;
  if constexpr (QUANT) {
    bool same = true;
    const float invs = hdmoe_q_inv_scale(q.shared_scale);
    if (q.shared_scale3 != q.shared_scale) ok13 = hdmoe_q_inv_scale(q.shared_scale3) == invs;
    for (int e = 0; e < E; ++e) {
      const float inv = hdmoe_q_inv_scale(q.scale_in.p[e]);
      same = same && inv == invs;
      if (q.scale_in3.p[e] != q.scale_in.p[e]) ok13 = ok13 && hdmoe_q_inv_scale(q.scale_in3.p[e]) == inv;
    }
    one_row = q.decide ? same : q.xq_routed == nullptr;
    with_shared = q.decide ? q.with_shared != 0 : q.xq_shared != nullptr;
    if (blockIdx.x == 0 && threadIdx.x == 0) {
      if (q.decide) *q.layout_flag = same ? 1 : 0;
      if (!ok13 && q.scale_check != nullptr) *q.scale_check = 1;
    }
  }
  // Up to TG tokens of the wave's walk per trip: one read of a weight slice serves them all, and the weight traffic
  // through the caches, E * D * 2 bytes per token otherwise, is what bounds this kernel. Each token's sums are formed
  // from the same operands in the same order as alone.
  constexpr int TG = GENERIC_TOKENS_PER_TRIP;
  for (int t = walk.first; t < t_end; t += TG * walk.step) {
    float logit[TG][E];
#pragma unroll
    for (int g = 0; g < TG; ++g)
#pragma unroll
      for (int e = 0; e < E; ++e) logit[g][e] = 0.0f;
    for (int u = lane; u < row16; u += 64) {
      uint4 xv[TG];
#pragma unroll
      for (int g = 0; g < TG; ++g) {
        const int tg = t + g * walk.step;
        xv[g] = x[(size_t)(tg < t_end ? tg : t) * row16 + u];   // past the end: the first token again, result dropped
      }
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const uint4 wv = wg[(size_t)e * row16 + u];
#pragma unroll
        for (int g = 0; g < TG; ++g) logit[g][e] = dot8<A>(xv[g], wv, logit[g][e]);
      }
    }
#pragma unroll
    for (int g = 0; g < TG; ++g) {
      const int tg = t + g * walk.step;
      if (tg >= t_end) break;
      int i0, i1;
      finish_token<E, A>(logit[g], lane, tg, idx, wout, i0, i1);
#pragma unroll
      for (int e = 0; e < E; ++e) cnt[e] += (i0 == e) + (i1 == e);
      if constexpr (QUANT) {
        const float bad = __builtin_nanf("");   // a cast that cannot serve w1 and w3 alike: NaN rows
        const float inv0 = hdmoe_q_uniform(ok13 ? hdmoe_q_inv_scale(q.scale_in.p[i0]) : bad);
        const float inv1 = hdmoe_q_uniform(ok13 ? hdmoe_q_inv_scale(q.scale_in.p[i1]) : bad);
        const float invs = hdmoe_q_uniform(ok13 ? hdmoe_q_inv_scale(q.shared_scale) : bad);
        for (int u = lane; u < row16; u += 64) {
          const uint4 xv = x[(size_t)tg * row16 + u];
          if (!one_row) {
            q.xq_routed[(size_t)(2 * tg) * row16 + u] = hdmoe_q_8(xv, inv0);
            q.xq_routed[(size_t)(2 * tg + 1) * row16 + u] = hdmoe_q_8(xv, inv1);
          }
          if (one_row || with_shared) q.xq_shared[(size_t)tg * row16 + u] = hdmoe_q_8(xv, invs);
        }
      }
    }
  }
  write_block_hist<E>(cnt, block_hist);
}

// which kernel a launch gets, as a function of the sizes and of what the kernel has to do besides routing
enum GateKernel { KERNEL_GENERIC, KERNEL_ROUTE, KERNEL_SPLIT, KERNEL_LN };
GateKernel gate_kernel_of(int D, int E, bool f16, bool with_cast, bool with_ln) {
  if (f16 || E > 4 || D != 2560) return KERNEL_GENERIC;
  return !with_cast ? KERNEL_ROUTE : (with_ln ? KERNEL_LN : KERNEL_SPLIT);
}
// tokens a block takes per trip, and resident blocks per CU
int gate_trip_tokens(GateKernel k) { return k == KERNEL_GENERIC ? WAVES_PER_BLOCK : (k == KERNEL_SPLIT ? ROW_WAVES / 2 : ROW_WAVES); }
int gate_resident_blocks(GateKernel k) { return HDMOE_NUM_CU * (k == KERNEL_GENERIC ? 3 : ROW_BLOCKS_PER_CU); }

template <int E>
int launch_gate(const void* x, const void* wg, int T, int D, int32_t* idx, void* w, const GateQuant* quant,
                int32_t* block_hist, hipStream_t s, const char* what, bool f16) {
  const bool ln = quant != nullptr && quant->mod_scale != nullptr;
  const GateKernel kernel = gate_kernel_of(D, E, f16, quant != nullptr, ln);
  if (ln && kernel != KERNEL_LN) return hdmoe_fail(HDMOE_E_SHAPE, "%s: the LayerNorm variant needs D = 2560 and E <= 4", what);
  if (f16 && quant) return hdmoe_fail(HDMOE_E_SHAPE, "%s: the fp8 cast takes bf16 activations", what);
  // with histograms: block ranges; without: waves strided over the tokens, at least two tokens per wave of the
  // generic kernel (more waves with fewer tokens each beat fewer waves with a full group of four: 29 against 31 us
  // at 8192 tokens, 8 experts, width 2048), and no more blocks than are resident at once
  const int tpb = block_hist != nullptr ? hdmoe_gate_tokens_per_block(T, D, E, quant != nullptr, ln) : 0;
  const int per_block = kernel == KERNEL_GENERIC ? 2 * WAVES_PER_BLOCK : gate_trip_tokens(kernel);
  int blocks = tpb > 0 ? (T + tpb - 1) / tpb : (T + per_block - 1) / per_block;
  if (tpb == 0 && blocks > gate_resident_blocks(kernel)) blocks = gate_resident_blocks(kernel);
  dim3 grid(blocks < 1 ? 1 : blocks), block((kernel == KERNEL_GENERIC ? WAVES_PER_BLOCK : ROW_WAVES) * 64);
  const uint4* xp = static_cast<const uint4*>(x);
  const uint4* wp = static_cast<const uint4*>(wg);
  uint16_t* wo = static_cast<uint16_t*>(w);
  GateQuant q;
  memset(&q, 0, sizeof(q));
  if (quant) q = *quant;
  constexpr int ER = E <= 4 ? E : 4;  // the register kernels are only instantiated for up to 4 experts
  switch (kernel) {
    case KERNEL_ROUTE:
      hipLaunchKernelGGL((gate_row_kernel<ER, 5, GATE_ROUTE>), grid, block, 0, s, xp, wp, T, tpb, idx, wo, block_hist, q);
      break;
    case KERNEL_SPLIT:
      hipLaunchKernelGGL((gate_row_kernel<ER, 5, GATE_SPLIT>), grid, block, 0, s, xp, wp, T, tpb, idx, wo, block_hist, q);
      break;
    case KERNEL_LN:
      hipLaunchKernelGGL((gate_row_kernel<ER, 5, GATE_LN>), grid, block, 0, s, xp, wp, T, tpb, idx, wo, block_hist, q);
      break;
    case KERNEL_GENERIC:
      if (f16)
        hipLaunchKernelGGL((gate_top2_generic_kernel<E, false, GateF16>), grid, block, 0, s, xp, wp, T, D, tpb, idx, wo,
                           block_hist, q);
      else if (quant)
        hipLaunchKernelGGL((gate_top2_generic_kernel<E, true>), grid, block, 0, s, xp, wp, T, D, tpb, idx, wo, block_hist, q);
      else
        hipLaunchKernelGGL((gate_top2_generic_kernel<E, false>), grid, block, 0, s, xp, wp, T, D, tpb, idx, wo, block_hist, q);
      break;
  }
  return hdmoe_check_launch(what);
}

int dispatch_gate(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E, int32_t* topk_idx,
                  void* topk_weight_bf16, const GateQuant* quant, int32_t* block_hist, hipStream_t s,
                  const char* what, bool f16 = false) {
  switch (E) {
#define HDMOE_GATE_CASE(n) \
  case n: return launch_gate<n>(x_bf16, gate_w_bf16, T, D, topk_idx, topk_weight_bf16, quant, block_hist, s, what, f16);
    HDMOE_GATE_CASE(2) HDMOE_GATE_CASE(3) HDMOE_GATE_CASE(4) HDMOE_GATE_CASE(5) HDMOE_GATE_CASE(6)
    HDMOE_GATE_CASE(7) HDMOE_GATE_CASE(8) HDMOE_GATE_CASE(9) HDMOE_GATE_CASE(10) HDMOE_GATE_CASE(11)
    HDMOE_GATE_CASE(12) HDMOE_GATE_CASE(13) HDMOE_GATE_CASE(14) HDMOE_GATE_CASE(15) HDMOE_GATE_CASE(16)
#undef HDMOE_GATE_CASE
    default: return hdmoe_fail(HDMOE_E_SHAPE, "%s: E=%d not in 2..16", what, E);
  }
}

// ---- LayerNorm (no affine) + adaLN modulation in front of the feed-forward -----------------------------
// n = bf16(LayerNorm(x)); out = bf16( bf16(n * bf16(1 + scale[b])) + shift[b] ), b = token / tokens_per_batch
// (/root/reference/comfy/ldm/hidream/model.py:430-431, 516-517). One token per wave, same lane/element mapping
// as the gate kernel; mean and variance are two passes over the registers with the same fixed fp32 order
// (per-lane ascending elements, then the xor butterfly), so the CPU checker can restate it bit for bit.
// The root is __builtin_sqrtf, which hipcc rounds correctly; __fsqrt_rn is the approximate native root here.
template <int NCHUNK>  // NCHUNK * 512 == D: row held in registers; 0: any D % 8 == 0, row re-read from cache
__global__ __launch_bounds__(WAVES_PER_BLOCK * 64) void ln_modulate_kernel(
    const uint4* __restrict__ x, const uint4* __restrict__ scale, const uint4* __restrict__ shift, int T, int D,
    int tokens_per_batch, float eps, uint4* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * WAVES_PER_BLOCK + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * WAVES_PER_BLOCK;
  const int row16 = D / 8;
  const float fD = (float)D;
  for (int t = wave; t < T; t += nwaves) {
    const uint4* xr = x + (size_t)t * row16;
    const size_t brow = (size_t)(t / tokens_per_batch) * row16;
    if constexpr (NCHUNK > 0) {
      uint4 v[NCHUNK];
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c) v[c] = xr[c * 64 + lane];
      float mean, rstd;
      ln_stats<NCHUNK>(v, fD, eps, mean, rstd);
#pragma unroll
      for (int c = 0; c < NCHUNK; ++c)
        out[(size_t)t * row16 + c * 64 + lane] =
            modulate8(v[c], scale[brow + c * 64 + lane], shift[brow + c * 64 + lane], mean, rstd);
    } else {
      float s = 0.0f;
      for (int u = lane; u < row16; u += 64) {
        float f[8];
        unpack8(xr[u], f);
#pragma unroll
        for (int j = 0; j < 8; ++j) s = s + f[j];
      }
      const float mean = __fdiv_rn(wave_sum(s), fD);
      float s2 = 0.0f;
      for (int u = lane; u < row16; u += 64) {
        float f[8];
        unpack8(xr[u], f);
#pragma unroll
        for (int j = 0; j < 8; ++j) { const float d = f[j] - mean; s2 = __builtin_fmaf(d, d, s2); }
      }
      const float rstd = __fdiv_rn(1.0f, __builtin_sqrtf(__fdiv_rn(wave_sum(s2), fD) + eps));
      for (int u = lane; u < row16; u += 64)
        out[(size_t)t * row16 + u] = modulate8(xr[u], scale[brow + u], shift[brow + u], mean, rstd);
    }
  }
}

}  // namespace

extern "C" int hdmoe_gate_top2(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E,
                               int32_t* topk_idx, void* topk_weight_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(gate_w_bf16);
  HDMOE_REQUIRE_PTR(topk_idx);
  HDMOE_REQUIRE_PTR(topk_weight_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_gate_top2: T=%d D=%d (D must be a positive multiple of 8)", T, D);
  if (T == 0) return HDMOE_OK;
  return dispatch_gate(x_bf16, gate_w_bf16, T, D, E, topk_idx, topk_weight_bf16, nullptr, nullptr,
                       static_cast<hipStream_t>(stream), "hdmoe_gate_top2");
}

extern "C" int hdmoe_gate_top2_f16(const void* x_f16, const void* gate_w_f16, int T, int D, int E, int32_t* topk_idx,
                                   void* topk_weight_f16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_f16);
  HDMOE_REQUIRE_PTR(gate_w_f16);
  HDMOE_REQUIRE_PTR(topk_idx);
  HDMOE_REQUIRE_PTR(topk_weight_f16);
  if (T < 0 || D <= 0 || D % 8 != 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_gate_top2_f16: T=%d D=%d (D must be a positive multiple of 8)", T, D);
  if (T == 0) return HDMOE_OK;
  return dispatch_gate(x_f16, gate_w_f16, T, D, E, topk_idx, topk_weight_f16, nullptr, nullptr,
                       static_cast<hipStream_t>(stream), "hdmoe_gate_top2_f16", true);
}

// Tokens per block of the gate kernels of the one-call layer, a pure function of the sizes and of the kernel
// (with_cast: fp8 experts; with_ln: LayerNorm + modulation inside the kernel). All blocks resident at once, each a
// whole number of trips. Very large T gets more blocks instead of more than 1024 tokens each (the dispatch's scatter
// pass handles one or several whole blocks per chunk, at most 1024 tokens).
int hdmoe_gate_tokens_per_block(int T, int D, int E, bool with_cast, bool with_ln) {
  const GateKernel kernel = gate_kernel_of(D, E, false, with_cast, with_ln);
  const int resident = gate_resident_blocks(kernel), unit = gate_trip_tokens(kernel);
  int tpb = (T + resident - 1) / resident;
  tpb = (tpb + unit - 1) / unit * unit;
  if (tpb < unit) tpb = unit;
  if (tpb > 1024) tpb = 1024;
  return tpb;
}

// Bytes of the per-block expert histograms the gate kernels can leave for the dispatch: enough for either kernel
// a layer of these sizes may get.
size_t hdmoe_gate_hist_bytes(int T, int D, int E, bool with_cast) {
  size_t most = 0;
  for (int ln = 0; ln < (with_cast ? 2 : 1); ++ln) {
    const int tpb = hdmoe_gate_tokens_per_block(T, D, E, with_cast, ln != 0);
    const size_t blocks = T > 0 ? ((size_t)T + tpb - 1) / tpb : 1;
    if (blocks > most) most = blocks;
  }
  return hdmoe_align_up(most * (size_t)E * sizeof(int32_t), 256);
}

// The same gate for the one-call layer, which also takes the histograms.
int hdmoe_launch_gate(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E, int32_t* topk_idx,
                      void* topk_weight_bf16, int32_t* block_hist, hipStream_t s, const char* what) {
  return dispatch_gate(x_bf16, gate_w_bf16, T, D, E, topk_idx, topk_weight_bf16, nullptr, block_hist, s, what);
}

// The gate of the one-call layer with fp8 experts: routing plus the token's three fp8 rows in one pass over x.
// Whether the gate + cast kernel can also do the block's LayerNorm + modulation in front of it.
bool hdmoe_gate_quant_takes_ln(int D, int E) { return D == 2560 && E <= 4; }

int hdmoe_launch_gate_quant(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E, int32_t* topk_idx,
                            void* topk_weight_bf16, const float* const* scale_input, const float* shared_scale,
                            void* xq_routed, void* xq_shared, hipStream_t s, const char* what,
                            const void* mod_scale = nullptr, const void* mod_shift = nullptr, int tokens_per_batch = 0,
                            float ln_eps = 0.0f, int32_t* block_hist = nullptr, const HdmoeGateScaleChecks* checks = nullptr) {
  GateQuant q;
  memset(&q, 0, sizeof(q));
  for (int e = 0; e < E && e < HDMOE_MAX_EXPERTS; ++e) q.scale_in3.p[e] = scale_input[e];  // nothing to compare
  q.shared_scale3 = shared_scale;
  if (checks != nullptr) {
    q.decide = checks->decide ? 1 : 0;
    q.with_shared = checks->with_shared ? 1 : 0;
    q.layout_flag = checks->layout_flag;
    q.scale_check = checks->scale_check;
    for (int e = 0; e < E && e < HDMOE_MAX_EXPERTS; ++e) q.scale_in3.p[e] = checks->scale_in3[e];
    q.shared_scale3 = checks->shared_scale3;
  }
  if (mod_scale != nullptr) {
    q.mod_scale = static_cast<const uint4*>(mod_scale);
    q.mod_shift = static_cast<const uint4*>(mod_shift);
    q.tokens_per_batch = tokens_per_batch;
    q.ln_eps = ln_eps;
  }
  for (int e = 0; e < E && e < HDMOE_MAX_EXPERTS; ++e) q.scale_in.p[e] = scale_input[e];
  q.shared_scale = shared_scale;
  q.xq_routed = static_cast<uint2*>(xq_routed);
  q.xq_shared = static_cast<uint2*>(xq_shared);
  return dispatch_gate(x_bf16, gate_w_bf16, T, D, E, topk_idx, topk_weight_bf16, &q, block_hist, s, what);
}

extern "C" int hdmoe_ln_modulate_bf16(const void* x_bf16, const void* scale_bf16, const void* shift_bf16, int T, int D,
                                      int tokens_per_batch, float eps, void* out_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(scale_bf16);
  HDMOE_REQUIRE_PTR(shift_bf16);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (T < 0 || D <= 0 || D % 8 != 0 || tokens_per_batch <= 0 || !(eps >= 0.0f))
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_ln_modulate_bf16: T=%d D=%d tokens_per_batch=%d eps=%g", T, D,
                      tokens_per_batch, (double)eps);
  if (T == 0) return HDMOE_OK;
  int blocks = (T + WAVES_PER_BLOCK - 1) / WAVES_PER_BLOCK;
  if (blocks > HDMOE_NUM_CU * 16) blocks = HDMOE_NUM_CU * 16;
  const dim3 grid(blocks), block(WAVES_PER_BLOCK * 64);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const uint4* xp = static_cast<const uint4*>(x_bf16);
  const uint4* sc = static_cast<const uint4*>(scale_bf16);
  const uint4* sh = static_cast<const uint4*>(shift_bf16);
  uint4* op = static_cast<uint4*>(out_bf16);
  if (D == 2560) hipLaunchKernelGGL(ln_modulate_kernel<5>, grid, block, 0, s, xp, sc, sh, T, D, tokens_per_batch, eps, op);
  else hipLaunchKernelGGL(ln_modulate_kernel<0>, grid, block, 0, s, xp, sc, sh, T, D, tokens_per_batch, eps, op);
  return hdmoe_check_launch("hdmoe_ln_modulate_bf16");
}
