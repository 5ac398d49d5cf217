/*
 * TEST INFRASTRUCTURE ONLY. CPU restatement, in plain C, of the integer/bit-level
 * parts of the HiDream MoE feed-forward as ComfyUI runs it. Only tests/,
 * __graft_entry__.smoke() and bench.py's cpu_baseline leg may load this; the
 * product (comfyui_amd/) never does.
 *
 * Reference followed (paths relative to /root/reference):
 *   gate      comfy/ldm/hidream/model.py:263-283  (F.linear -> softmax -> top-2 of E, not renormalised)
 *   dispatch  comfy/ldm/hidream/model.py:312-318  (flat slot p = 2t+s; expert i takes rows with idx==i in ascending p)
 *   combine   comfy/ldm/hidream/model.py:319-324  ((y.view(T,2,D) * w.unsqueeze(-1)).sum(1) + shared)
 *   fp8 cast  comfy/ops.py:337-343                (tensor.to(float8_e4m3fn): RNE, no saturation)
 *
 * The arithmetic of all of these lives in PyTorch (unpinned in requirements.txt:4;
 * 2.10.0 in this image); the reference holds no golden vectors for them, so each
 * function here is pinned by tests/test_oracle_*.py against closed forms, brute
 * force and the torch library routines named in those tests.
 *
 * ref_gate_top2 fixes ONE summation order for the fp32 dot products (the order the
 * HIP gate kernel uses: 64 partial sums over 8-element groups strided by 512
 * elements, then a pairwise tree 32,16,8,4,2,1) and one exp() (a fixed fp32
 * polynomial), so that the kernel can be compared bit for bit. Its agreement with
 * torch's own summation order is checked statistically in the tests.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

/* built with -ffp-contract=off (see Makefile): a*b+c is never fused unless fmaf() says so */


static float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }
static uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }

static float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* round-to-nearest-even fp32 -> bf16 (finite inputs and NaN) */
static uint16_t f32_to_bf16(float f) {
  uint32_t u = f32_bits(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
  uint32_t lower = u & 0xffffu, keep = u >> 16;
  if (lower > 0x8000u || (lower == 0x8000u && (keep & 1u))) keep += 1u;
  return (uint16_t)keep;
}

/* IEEE binary16 <-> fp32 by the definition: 1 sign, 5 exponent (bias 15), 10 mantissa bits, subnormals m * 2^-24,
 * exponent 31 = inf / NaN. Encode rounds to nearest even through ldexp/nearbyint arithmetic on the value (not bit
 * tricks), overflows to infinity at 65520 and above. Pinned against torch's own conversion in the tests (all 65536
 * patterns decoded, random and boundary values encoded). */
static float f16_to_f32(uint16_t h) {
  int s = h >> 15, e = (h >> 10) & 31, m = h & 1023;
  float v;
  if (e == 31) v = m ? NAN : INFINITY;
  else if (e == 0) v = ldexpf((float)m, -24);
  else v = ldexpf(1.0f + (float)m / 1024.0f, e - 15);
  return s ? -v : v;
}

static uint16_t f32_to_f16(float f) {
  uint16_t sign = (f32_bits(f) >> 31) ? 0x8000u : 0;
  if (isnan(f)) return (uint16_t)(sign | 0x7e00u);
  double a = fabs((double)f);
  if (a >= 65520.0) return (uint16_t)(sign | 0x7c00u);          /* the midpoint above 65504 rounds to infinity */
  if (a < ldexp(1.0, -14)) {                                    /* subnormal range: multiples of 2^-24 */
    double q = nearbyint(ldexp(a, 24));                         /* default rounding mode: to nearest even */
    return (uint16_t)(sign | (uint16_t)q);                      /* q == 1024 is the smallest normal, same bits */
  }
  int ex;
  double fr = frexp(a, &ex);                                    /* a = fr * 2^ex, fr in [0.5, 1) */
  double q = nearbyint(ldexp(fr, 11));                          /* 11 significant bits: 1024 .. 2048 */
  if (q == 2048.0) { q = 1024.0; ex += 1; }
  int e = ex - 1 + 15;
  if (e >= 31) return (uint16_t)(sign | 0x7c00u);
  return (uint16_t)(sign | (uint16_t)(e << 10) | (uint16_t)((int)q - 1024));
}

void ref_f16_decode(const uint16_t* in, float* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = f16_to_f32(in[i]); }
void ref_f16_encode(const float* in, uint16_t* out, int64_t n) { for (int64_t i = 0; i < n; ++i) out[i] = f32_to_f16(in[i]); }

/* ---- float8_e4m3fn ---------------------------------------------------------- */

/* closed form: (-1)^s * 2^(e-7) * (1 + m/8), e==0 -> m * 2^-9, 0x7F/0xFF NaN */
void ref_e4m3fn_decode_table(float out[256]) {
  for (int b = 0; b < 256; ++b) {
    int s = b >> 7, e = (b >> 3) & 15, m = b & 7;
    float v;
    if (e == 15 && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf(1.0f + (float)m / 8.0f, e - 7);
    out[b] = s ? -v : v;
  }
}

/* Nearest-value search over the 127 finite magnitudes, ties to the even code,
 * overflow past the midpoint above 448 (i.e. > 464) -> NaN, NaN -> NaN.
 * Deliberately a search, not bit tricks, so it shares nothing with the kernels. */
void ref_e4m3fn_encode(const float* in, uint8_t* out, int64_t n) {
  float tab[256];
  ref_e4m3fn_decode_table(tab);
  for (int64_t i = 0; i < n; ++i) {
    float f = in[i];
    uint8_t sign = (f32_bits(f) >> 31) ? 0x80 : 0;
    float a = fabsf(f);
    if (isnan(f) || a > 464.0f) { out[i] = sign | 0x7f; continue; }
    int lo = 0, hi = 126; /* tab[0..126] ascending finite magnitudes, tab[126] = 448 */
    while (lo < hi) { int mid = (lo + hi + 1) / 2; if (tab[mid] <= a) lo = mid; else hi = mid - 1; }
    int code = lo;
    if (lo < 126) {
      double dlo = (double)a - (double)tab[lo], dhi = (double)tab[lo + 1] - (double)a;
      if (dhi < dlo || (dhi == dlo && (lo & 1))) code = lo + 1;
    } else {
      /* between 448 and 464: 464 itself is the tie and goes to the even code 0x7E = 448 */
      code = 126;
    }
    out[i] = sign | (uint8_t)code;
  }
}

/* ---- gate ------------------------------------------------------------------- */

/* exp(x) for x <= 0, fixed fp32 evaluation order (range reduction by ln2 split in
 * two, degree-5 polynomial, exponent added through the bit pattern). */
static float ref_exp_neg(float x) {
  if (x < -80.0f) x = -80.0f;
  float n = nearbyintf(x * 1.44269504088896341f);
  float r = fmaf(n, -0.693359375f, x);
  r = fmaf(n, 2.12194440e-4f, r);
  float p = 1.9875691500e-4f;
  p = fmaf(p, r, 1.3981999507e-3f);
  p = fmaf(p, r, 8.3334519073e-3f);
  p = fmaf(p, r, 4.1665795894e-2f);
  p = fmaf(p, r, 1.6666665459e-1f);
  p = fmaf(p, r, 5.0000001201e-1f);
  float z = r * r;
  float y = fmaf(p, z, r);
  y = y + 1.0f;
  return bits_f32(f32_bits(y) + ((uint32_t)(int32_t)n << 23));
}

/* x [T,D] bf16, wg [E,D] bf16 -> idx [T,2] int32 (slot 0 = larger score, ties to
 * the lower expert index), w [T,2] bf16 scores, optional logits/scores [T,E] bf16.
 * D must be a multiple of 8, 2 <= E <= 16. Returns 0, or -1 on bad arguments. */
static int gate_top2_fmt(const uint16_t* x, const uint16_t* wg, int T, int D, int E,
                         int32_t* idx, uint16_t* w, uint16_t* logits_out, uint16_t* scores_out,
                         float (*bf16_to_f32)(uint16_t), uint16_t (*f32_to_bf16)(float)) {
  /* the two parameters shadow the bf16 conversions: the body below reads the same for either 16-bit format */
  if (D % 8 != 0 || E < 2 || E > 16 || T < 0) return -1;
  for (int t = 0; t < T; ++t) {
    const uint16_t* xr = x + (size_t)t * D;
    float logit[16] = {0}, score[16] = {0};
    for (int e = 0; e < E; ++e) {
      const uint16_t* wr = wg + (size_t)e * D;
      float lane[64];
      for (int l = 0; l < 64; ++l) {
        float acc = 0.0f;
        for (int base = l * 8; base < D; base += 512)
          for (int j = 0; j < 8; ++j)
            acc = fmaf(bf16_to_f32(xr[base + j]), bf16_to_f32(wr[base + j]), acc);
        lane[l] = acc;
      }
      for (int off = 32; off >= 1; off >>= 1)
        for (int l = 0; l < off; ++l) lane[l] = lane[l] + lane[l + off];
      logit[e] = bf16_to_f32(f32_to_bf16(lane[0]));
    }
    float mx = logit[0];
    for (int e = 1; e < E; ++e) mx = logit[e] > mx ? logit[e] : mx;
    float ex[16], sum = 0.0f;
    for (int e = 0; e < E; ++e) { ex[e] = ref_exp_neg(logit[e] - mx); sum = sum + ex[e]; }
    for (int e = 0; e < E; ++e) score[e] = bf16_to_f32(f32_to_bf16(ex[e] / sum));
    int i0 = 0;
    for (int e = 1; e < E; ++e) if (score[e] > score[i0]) i0 = e;
    int i1 = -1;
    for (int e = 0; e < E; ++e) { if (e == i0) continue; if (i1 < 0 || score[e] > score[i1]) i1 = e; }
    idx[2 * t] = i0; idx[2 * t + 1] = i1;
    w[2 * t] = f32_to_bf16(score[i0]); w[2 * t + 1] = f32_to_bf16(score[i1]);
    if (logits_out) for (int e = 0; e < E; ++e) logits_out[(size_t)t * E + e] = f32_to_bf16(logit[e]);
    if (scores_out) for (int e = 0; e < E; ++e) scores_out[(size_t)t * E + e] = f32_to_bf16(score[e]);
  }
  return 0;
}

int ref_gate_top2(const uint16_t* x, const uint16_t* wg, int T, int D, int E,
                  int32_t* idx, uint16_t* w, uint16_t* logits_out, uint16_t* scores_out) {
  return gate_top2_fmt(x, wg, T, D, E, idx, w, logits_out, scores_out, bf16_to_f32, f32_to_bf16);
}

/* the same gate on fp16 tensors: x, wg, w, logits and scores fp16, the two roundings to fp16 */
int ref_gate_top2_f16(const uint16_t* x, const uint16_t* wg, int T, int D, int E,
                      int32_t* idx, uint16_t* w, uint16_t* logits_out, uint16_t* scores_out) {
  return gate_top2_fmt(x, wg, T, D, E, idx, w, logits_out, scores_out, f16_to_f32, f32_to_f16);
}

/* ---- dispatch --------------------------------------------------------------- */

/* flat[p] for p in [0, n): expert of flat slot p (p = K*t + s). Stable counting
 * sort: perm[r] = flat slot held by sorted row r, inv_perm[p] = sorted row of slot p,
 * offsets = exclusive scan of counts (E+1 entries). */
int ref_dispatch(const int32_t* flat, int64_t n, int E, int32_t* counts, int32_t* offsets,
                 int32_t* perm, int32_t* inv_perm) {
  for (int e = 0; e < E; ++e) counts[e] = 0;
  for (int64_t p = 0; p < n; ++p) {
    if (flat[p] < 0 || flat[p] >= E) return -1;
    counts[flat[p]]++;
  }
  offsets[0] = 0;
  for (int e = 0; e < E; ++e) offsets[e + 1] = offsets[e] + counts[e];
  int32_t* cur = (int32_t*)malloc(sizeof(int32_t) * (size_t)E);
  for (int e = 0; e < E; ++e) cur[e] = offsets[e];
  for (int64_t p = 0; p < n; ++p) {
    int32_t r = cur[flat[p]]++;
    perm[r] = (int32_t)p;
    inv_perm[p] = r;
  }
  free(cur);
  return 0;
}

/* ---- combine ---------------------------------------------------------------- */

/* adaLN prologue of the feed-forward branch (model.py:430-431, 516-517):
 *   n = bf16(LayerNorm(x[t], eps))   (no affine, biased variance, fp32 statistics)
 *   out[t] = bf16( bf16(n * bf16(1 + scale[b])) + shift[b] ),  b = t / tokens_per_batch.
 * Mean and variance are two passes in ONE fixed fp32 order (the HIP kernel's: 64 partial sums over
 * 8-element groups strided by 512 elements, then the pairwise tree), so the kernel compares bit for
 * bit; agreement with torch's own layer_norm is checked in the tests to one bf16 step. */
static float tree64(float* lane) {
  for (int off = 32; off >= 1; off >>= 1)
    for (int l = 0; l < off; ++l) lane[l] = lane[l] + lane[l + off];
  return lane[0];
}

int ref_ln_modulate(const uint16_t* x, const uint16_t* scale, const uint16_t* shift, int T, int D,
                    int tokens_per_batch, float eps, uint16_t* out) {
  if (D % 8 != 0 || D <= 0 || T < 0 || tokens_per_batch <= 0) return -1;
  for (int t = 0; t < T; ++t) {
    const uint16_t* xr = x + (size_t)t * D;
    const uint16_t* sc = scale + (size_t)(t / tokens_per_batch) * D;
    const uint16_t* sh = shift + (size_t)(t / tokens_per_batch) * D;
    float lane[64];
    for (int l = 0; l < 64; ++l) {
      float acc = 0.0f;
      for (int base = l * 8; base < D; base += 512)
        for (int j = 0; j < 8; ++j) acc = acc + bf16_to_f32(xr[base + j]);
      lane[l] = acc;
    }
    const float mean = tree64(lane) / (float)D;
    for (int l = 0; l < 64; ++l) {
      float acc = 0.0f;
      for (int base = l * 8; base < D; base += 512)
        for (int j = 0; j < 8; ++j) {
          const float d = bf16_to_f32(xr[base + j]) - mean;
          acc = fmaf(d, d, acc);
        }
      lane[l] = acc;
    }
    const float rstd = 1.0f / sqrtf(tree64(lane) / (float)D + eps);
    for (int d = 0; d < D; ++d) {
      const float n = bf16_to_f32(f32_to_bf16((bf16_to_f32(xr[d]) - mean) * rstd));
      const float m = bf16_to_f32(f32_to_bf16(1.0f + bf16_to_f32(sc[d])));
      const float p = bf16_to_f32(f32_to_bf16(n * m));
      out[(size_t)t * D + d] = f32_to_bf16(p + bf16_to_f32(sh[d]));
    }
  }
  return 0;
}

/* Gated residual epilogue (model.py:432-433, 518-523): out = bf16( bf16(gate[b] * y[t]) + residual[t] ). */
void ref_gated_residual(const uint16_t* y, const uint16_t* gate, const uint16_t* residual, int T, int D,
                        int tokens_per_batch, uint16_t* out) {
  for (int t = 0; t < T; ++t) {
    const uint16_t* g = gate + (size_t)(t / tokens_per_batch) * D;
    for (int d = 0; d < D; ++d) {
      const size_t i = (size_t)t * D + d;
      const float p = bf16_to_f32(f32_to_bf16(bf16_to_f32(g[d]) * bf16_to_f32(y[i])));
      out[i] = f32_to_bf16(p + bf16_to_f32(residual[i]));
    }
  }
}

/* y_sorted [2T,D] bf16 (row r = expert output of flat slot perm[r]); w [T,2] bf16;
 * shared [T,D] bf16 or NULL. out[t] = bf16( bf16( f32(bf16(y0*w0)) + f32(bf16(y1*w1)) ) + shared[t] )
 * which is how a bf16 `(y*w).sum(1)` then `+ shared` rounds (model.py:319,324). */
void ref_combine(const uint16_t* y_sorted, const int32_t* inv_perm, const uint16_t* w,
                 const uint16_t* shared, int T, int D, uint16_t* out) {
  for (int t = 0; t < T; ++t) {
    const uint16_t* y0 = y_sorted + (size_t)inv_perm[2 * t] * D;
    const uint16_t* y1 = y_sorted + (size_t)inv_perm[2 * t + 1] * D;
    float w0 = bf16_to_f32(w[2 * t]), w1 = bf16_to_f32(w[2 * t + 1]);
    for (int d = 0; d < D; ++d) {
      float a = bf16_to_f32(f32_to_bf16(bf16_to_f32(y0[d]) * w0));
      float b = bf16_to_f32(f32_to_bf16(bf16_to_f32(y1[d]) * w1));
      float s = bf16_to_f32(f32_to_bf16(a + b));
      if (shared) s = s + bf16_to_f32(shared[(size_t)t * D + d]);
      out[(size_t)t * D + d] = f32_to_bf16(s);
    }
  }
}

/* ---- stochastic rounding to float8_e4m3fn (float.py:14-67, ops.py:419-426) ---------------------- */

/* Philox4x32-10 (Salmon et al., SC'11), restated here so the checker shares no code with the kernels.
 * Pinned by the paper's known-answer vectors in the tests. */
void ref_philox4x32_10(const uint32_t ctr_in[4], const uint32_t key_in[2], uint32_t out[4]) {
  uint32_t c[4] = {ctr_in[0], ctr_in[1], ctr_in[2], ctr_in[3]};
  uint32_t k[2] = {key_in[0], key_in[1]};
  for (int round = 0; round < 10; ++round) {
    uint64_t a = 0xD2511F53ull * (uint64_t)c[0];
    uint64_t b = 0xCD9E8D57ull * (uint64_t)c[2];
    uint32_t n[4];
    n[0] = (uint32_t)(b >> 32) ^ c[1] ^ k[0];
    n[1] = (uint32_t)(b & 0xffffffffu);
    n[2] = (uint32_t)(a >> 32) ^ c[3] ^ k[1];
    n[3] = (uint32_t)(a & 0xffffffffu);
    memcpy(c, n, sizeof(c));
    k[0] += 0x9E3779B9u;
    k[1] += 0xBB67AE85u;
  }
  memcpy(out, c, sizeof(c));
}

/* fp32 -> nearest float16 value (round to nearest even), returned as fp32; overflow -> inf */
static float round_to_f16(float f) {
  if (f != f) return f;
  float a = fabsf(f);
  if (a >= 65520.0f) return copysignf(INFINITY, f);
  if (a == 0.0f) return f;
  int e;
  (void)frexpf(a, &e);                 /* a = m * 2^e, m in [0.5,1) */
  int lsb = (e - 1) - 10;              /* exponent of the last kept bit of a normal float16 */
  if (lsb < -24) lsb = -24;            /* subnormal float16: fixed step 2^-24 */
  float q = nearbyintf(ldexpf(a, -lsb)); /* default rounding mode: to nearest, ties to even */
  return copysignf(ldexpf(q, lsb), f);
}

/* The procedure of float.py with the uniform number u in [0,1) passed in. Returns the e4m3fn value as fp32. */
static float stochastic_round_value(float h, float u) {
  if (h != h) return h;
  float a = fabsf(h);
  if (a == 0.0f) return 0.0f;
  float exponent = floorf(log2f(a)) + 7.0f;       /* exact: log2f is exact on powers of two and monotone */
  if (isinf(a)) exponent = 15.0f;
  if (exponent < 0.0f) exponent = 0.0f;
  if (exponent > 15.0f) exponent = 15.0f;
  float pos, value;
  if (exponent != 0.0f) {
    pos = (a / ldexpf(1.0f, (int)exponent - 7) - 1.0f) * 8.0f;
    value = ldexpf(1.0f, (int)exponent - 7) * (1.0f + floorf(pos + u) / 8.0f);
  } else {
    pos = a / ldexpf(1.0f, -9);
    value = ldexpf(1.0f, -6) * (floorf(pos + u) / 8.0f);
  }
  if (!(value <= 448.0f)) value = 448.0f;
  return copysignf(value, h);
}

/* src [n] fp32, *scale (NULL = 1) -> out [n] e4m3fn codes. src_is_bf16: src holds bf16 values (as fp32) and the
 * division is a bf16 tensor division (scale and quotient rounded to bf16). */
void ref_stochastic_round_e4m3fn(const float* src, int64_t n, const float* scale, uint64_t seed, int src_is_bf16,
                                 uint8_t* out) {
  const uint32_t key[2] = {(uint32_t)seed, (uint32_t)(seed >> 32)};
  float s = scale ? *scale : 1.0f;
  if (src_is_bf16) s = bf16_to_f32(f32_to_bf16(s));
  for (int64_t i = 0; i < n; ++i) {
    const uint64_t g = (uint64_t)i >> 2;
    const uint32_t ctr[4] = {(uint32_t)g, (uint32_t)(g >> 32), 0u, 0u};
    uint32_t r[4];
    ref_philox4x32_10(ctr, key, r);
    const float u = (float)(r[i & 3] >> 8) * (1.0f / 16777216.0f);
    float x = src[i] / s;
    if (src_is_bf16) x = bf16_to_f32(f32_to_bf16(x));
    const float v = stochastic_round_value(round_to_f16(x), u);
    uint8_t code;
    ref_e4m3fn_encode(&v, &code, 1);                 /* v is representable: the search returns its code */
    if (v == 0.0f) code = (x == 0.0f || !signbit(v)) ? 0x00 : 0x80;
    out[i] = code;
  }
}
