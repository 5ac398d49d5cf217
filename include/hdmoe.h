/*
 * libhdmoe -- C ABI of the MI355X (gfx950) implementation of the HiDream
 * mixture-of-experts SwiGLU feed-forward.
 *
 * The reference (ComfyUI v0.3.64, all Python) has no FFI for this path; what each
 * entry point replaces is the torch call sequence at the cited reference lines
 * (paths relative to the reference root).
 *
 * Conventions
 *   - every pointer named *_dev / documented "device" is HIP device memory owned by
 *     the caller; "host array" means an ordinary host pointer to E entries that is
 *     only read during the call;
 *   - all matrices are row-major and contiguous; weights are [out_features, in_features]
 *     exactly as torch.nn.Linear stores them;
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued on it and the
 *     call returns without synchronising; nothing is allocated, so calls on different
 *     streams may overlap;
 *   - the only state the library keeps between calls: the thread-local error message, and per device one flag per
 *     GEMM kernel variant recording that hipFuncSetAttribute (the opt-in for more than 64 KiB of dynamic LDS) has
 *     been called for it on that device, plus the device address of the built-in buffer of hdmoe_dispatch_static;
 *   - two process-wide switches choose between kernels with the same results bit for bit (hdmoe_set_kernel_form
 *     below); they start from the environment variables HDMOE_SWIGLU4W / HDMOE_LIGHT, read once at first use;
 *   - return value 0 = enqueued; negative = HDMOE_E_* and nothing was enqueued;
 *     hdmoe_last_error() gives a thread-local message for the last failure;
 *   - scale pointers (float*, device) address the fp32 scalar Parameters
 *     `scale_weight` / `scale_input` of a scaled-fp8 Linear (comfy/ops.py:388-397);
 *     a NULL scale_input means "Parameter is None": the input is clamped to +-448
 *     and cast, with scale 1 (comfy/ops.py:337-340). The caller's input is never
 *     modified (the reference clamps it in place).
 */
#ifndef HDMOE_H
#define HDMOE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define HDMOE_VERSION 114

#define HDMOE_OK 0
#define HDMOE_E_NULL (-1)      /* required pointer is NULL */
#define HDMOE_E_SHAPE (-2)     /* unsupported or inconsistent sizes */
#define HDMOE_E_WORKSPACE (-3) /* workspace too small or misaligned */
#define HDMOE_E_LAUNCH (-4)    /* HIP reported a launch error */

#define HDMOE_MAX_EXPERTS 16
#define HDMOE_TOPK 2

/* weight storage of the Linear layers */
#define HDMOE_W_BF16 0
#define HDMOE_W_E4M3FN 1
/* fp16 weights with fp16 activations, bias and outputs: hdmoe_linear_bias only (and the *_f16 entry points below) */
#define HDMOE_W_F16 2

typedef void* hdmoe_stream_t;

int hdmoe_version(void);
const char* hdmoe_last_error(void);

/* Kernel-form switches. No counterpart in the reference: both choose between kernels of this library whose results are
 * the same bit for bit, for tests that compare the forms and for measurements. Process-wide; a call in flight on
 * another thread sees the old or the new value. A HIP graph keeps the kernels that were captured.
 *   HDMOE_FORM_SWIGLU4W: the fp8 gate/up contraction has an 8-wave kernel (256- or 320-token tiles) and a 4-wave one
 *     (one wave per SIMD, 256-token tiles, a tile's SiLU*mul epilogue issued between the MFMAs of the next tile; needs
 *     K a multiple of 256 and at least 2048, and scale_in2). AUTO: the 4-wave kernel runs where the 320-token tile
 *     would not be used (up to about 5000 tokens for HiDream's sizes; it is 2-3 % faster there and 1-2 % slower
 *     above). NEVER / ALWAYS (whenever the shapes allow).
 *   HDMOE_FORM_LIGHT: the 8-wave kernels (gate/up and down) have a form whose K loop skips the 32-token blocks of a
 *     tile that hold no rows. AUTO: it runs when every segment is one tile and the experts' tiles are half empty on
 *     average (rows per expert <= 128 and shared rows <= 256: up to 256 tokens for HiDream's sizes; 3-12 % faster
 *     there, slower above). NEVER (also keeps 16-bit weights off the three-stage kernels those sizes take) / ALWAYS
 *     (fp8).
 * Initial values: the environment variables HDMOE_SWIGLU4W / HDMOE_LIGHT, read once ("0" = NEVER, anything else =
 * ALWAYS, unset = AUTO). hdmoe_get_kernel_form returns the current value. */
#define HDMOE_FORM_SWIGLU4W 0
#define HDMOE_FORM_LIGHT 1
#define HDMOE_NUM_FORMS 2
#define HDMOE_FORM_AUTO (-1)
#define HDMOE_FORM_NEVER 0
#define HDMOE_FORM_ALWAYS 1
int hdmoe_set_kernel_form(int which, int value);
int hdmoe_get_kernel_form(int which);

/* Name of the kernel that the gate/up contraction of a whole layer (T tokens, E routed experts top-2, shared expert
 * if Hs > 0; has_scale_in2: the w2 Linears carry a scale_input) runs on under the current switches, for reports that
 * name the dominant kernel; "" for sizes the layer does not take. No counterpart in the reference. */
const char* hdmoe_gate_up_kernel_name(int weight_dtype, int T, int E, int D, int H, int Hs, int has_scale_in2);

/* ---- stage entry points ------------------------------------------------------ */

/* MoEGate.forward, comfy/ldm/hidream/model.py:263-283 (F.linear :268, softmax :270,
 * topk k=2 :275, no renormalisation :253). x [T,D] bf16, gate_w [E,D] bf16.
 * Writes topk_idx [T,2] int32 and topk_weight [T,2] bf16; slot 0 holds the larger
 * score, equal scores go to the lower expert index. Logits and scores are rounded
 * to bf16 between the three steps as the three torch kernels do.
 * D % 8 == 0, 2 <= E <= 16. The same gate serves comfy/ldm/hunyuan3dv2_1/hunyuandit.py:73-112 (E = 6 or 8). */
int hdmoe_gate_top2(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E,
                    int32_t* topk_idx, void* topk_weight_bf16, hdmoe_stream_t stream);

/* The same gate on fp16 tensors (x, gate_w, topk_weight fp16; logits and scores rounded to fp16 between the steps):
 * the dtype comfy/supported_models_base.py:46 lists first and model_management.unet_dtype picks for
 * comfy/ldm/hunyuan3dv2_1/hunyuandit.py:73-112 on a device with fp16 support. */
int hdmoe_gate_top2_f16(const void* x_f16, const void* gate_w_f16, int T, int D, int E,
                        int32_t* topk_idx, void* topk_weight_f16, hdmoe_stream_t stream);

/* Optional renormalisation of the two gate weights, comfy/ldm/hidream/model.py:277-280 (`norm_topk_prob`, off in
 * HiDream): out[t, s] = bf16( w[t, s] / bf16( bf16(w[t,0] + w[t,1]) + 1e-20 ) ), the rounding points of the three torch
 * ops on bf16 tensors. topk_weight and out are [T, 2] bf16 (out may be topk_weight). */
int hdmoe_renorm_top2_bf16(const void* topk_weight_bf16, int T, void* out_bf16, hdmoe_stream_t stream);

/* Token dispatch, comfy/ldm/hidream/model.py:313-318: the boolean-mask gathers
 * `x[flat_topk_idx == i]` for i = 0..E-1 select flat slots p = 2t+s in ascending p,
 * i.e. a stable sort of the flat expert ids. Writes counts [E], offsets [E+1]
 * (exclusive scan), perm [2T] (sorted row -> flat slot) and inv_perm [2T]
 * (flat slot -> sorted row), all int32 device arrays.
 * workspace: hdmoe_dispatch_workspace_bytes(T, E) bytes, 256-byte aligned. */
size_t hdmoe_dispatch_workspace_bytes(int T, int E);
int hdmoe_dispatch(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                   int32_t* perm, int32_t* inv_perm, void* workspace, size_t workspace_bytes,
                   hdmoe_stream_t stream);

/* The same dispatch for callers that cannot allocate device memory or carry a workspace (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc). It has no counterpart in the reference. The
 * per-chunk histograms that hdmoe_dispatch keeps in its workspace live in a 64 KiB device array inside the library
 * image instead (one copy per GPU, held until the process ends); the call allocates nothing. T is limited to
 * hdmoe_dispatch_static_max_tokens(E) (1 048 576 tokens at E = 16, more for fewer experts, capped by the int32 slot
 * range); beyond that the call returns HDMOE_E_WORKSPACE and enqueues nothing. All calls on one GPU share the array:
 * two calls whose kernels may overlap on the same GPU (different streams) race; calls on one stream do not. The
 * first call on a device looks the array's device address up (hipGetSymbolAddress, no allocation). */
int hdmoe_dispatch_static_max_tokens(int E);
int hdmoe_dispatch_static(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                          int32_t* perm, int32_t* inv_perm, hdmoe_stream_t stream);

/* Activation quantisation of fp8_linear, comfy/ops.py:337-343:
 * out = e4m3fn( bf16( x * bf16(1/scale_input) ) ), no saturation (|v| > 464 -> NaN);
 * scale_input == NULL: out = e4m3fn(clamp(x, -448, 448)).
 * x [rows,D] bf16 -> out [rows,D] bytes. D % 8 == 0. */
int hdmoe_quant_fp8(const void* x_bf16, int64_t rows, int D, const float* scale_input_dev,
                    void* out_fp8, hdmoe_stream_t stream);

/* Same quantisation fused with the gather of model.py:315,318: sorted row r takes
 * token perm[r] / 2 and the scale_input of the expert whose segment
 * [offsets[e], offsets[e+1]) holds r. scale_input: host array of E device pointers
 * (entries may be NULL). a_fp8 [2T,D]. */
int hdmoe_quant_permute_fp8(const void* x_bf16, const int32_t* perm, const int32_t* offsets,
                            int T, int D, int E, const float* const* scale_input,
                            void* a_fp8, hdmoe_stream_t stream);

/* bf16 gather of model.py:315,318 for bf16 weights: a[r] = x[perm[r] / 2]. Rows are copied as bytes, so any 16-bit
 * element type (fp16) goes through it unchanged. */
int hdmoe_permute_bf16(const void* x_bf16, const int32_t* perm, int T, int D, void* a_bf16,
                       hdmoe_stream_t stream);

/* One group of rows of a grouped GEMM: an expert (or the shared expert). */
typedef struct hdmoe_ffn_weights {
  const void* w1; /* [H,D] */
  const void* w2; /* [D,H] */
  const void* w3; /* [H,D] */
  /* fp8 only (ignored for bf16 weights): device fp32 scalars */
  const float* scale_w1;
  const float* scale_w2;
  const float* scale_w3;
  const float* scale_in1; /* scale_input of w1 */
  const float* scale_in2; /* scale_input of w2 */
  const float* scale_in3; /* scale_input of w3 */
  /* w1 and w3 read the same input, which the fused kernels quantise once, with scale_in1: the two scale_inputs must
   * give the same cast factor bf16(1 / scale_input). The host cannot compare device scalars without synchronising, so
   * the entry points accept scale_in1 == scale_in3 as pointers (both NULL included) and, for two different non-NULL
   * pointers, only a caller that sets this field to nonzero, asserting that the two values are equal; anything else
   * is HDMOE_E_SHAPE. The kernel that casts compares the two factors on the device and writes NaN instead of a cast
   * made with the wrong one (hdmoe_moe_ffn, hdmoe_ffn_swiglu). Each Linear's own scale_input value enters its
   * output scale. */
  int same_scale_in13;
} hdmoe_ffn_weights;

/* First half of FeedForwardSwiGLU.forward (model.py:238) for every expert at once:
 *   h[r] = quant2( bf16(silu(bf16(w1 a[r]))) * bf16(w3 a[r]) )       r in expert e's segment
 * with each Linear evaluated as fp8_linear (ops.py:345-348: fp32 accumulation of
 * fp8 x fp8 products, times scale_in*scale_w, rounded to bf16), and quant2 the
 * activation quantisation of the following w2 Linear (scale_in2), so h is e4m3fn.
 * For bf16 weights every Linear is bf16 x bf16 with fp32 accumulation and h is bf16.
 * a [rows_total,D] (e4m3fn or bf16, rows sorted by expert), offsets [E+1] device,
 * h [rows_total,H]. D % 128 == 0 (fp8) or D % 64 == 0 (bf16); H % 128 == 0. */
int hdmoe_grouped_swiglu(int weight_dtype, const void* a, const int32_t* offsets, int rows_total,
                         int E, int D, int H, const hdmoe_ffn_weights* experts, void* h,
                         hdmoe_stream_t stream);

/* Second half: y[r] = bf16(w2 h[r]) per expert segment. h [rows_total,H], y [rows_total,D] bf16.
 * H % 128 == 0 (fp8) or H % 64 == 0 (bf16); D % 256 == 0. */
int hdmoe_grouped_down(int weight_dtype, const void* h, const int32_t* offsets, int rows_total,
                       int E, int H, int D, const hdmoe_ffn_weights* experts, void* y_bf16,
                       hdmoe_stream_t stream);

/* One Linear without bias on already-prepared activations:
 *   fp8:  out = bf16( (a_fp8 . w_fp8^T) * scale_in * scale_w )   (fp8_linear, ops.py:345-348;
 *         scale_in NULL = 1)
 *   bf16: out = bf16( a_bf16 . w_bf16^T )                        (Linear, ops.py:107-115)
 * a [rows,K], w [N,K], out [rows,N] bf16. K % 128 == 0 (fp8) / K % 64 == 0 (bf16); N % 256 == 0. */
int hdmoe_linear(int weight_dtype, const void* a, int rows, int K, int N, const void* w,
                 const float* scale_w_dev, const float* scale_in_dev, void* out_bf16,
                 hdmoe_stream_t stream);

/* The same Linear with a bias (bias_bf16 [N]; NULL = hdmoe_linear): the bias joins the fp32 result before the one
 * rounding, as F.linear does (ops.py:107-115) and as the scaled matrix multiply of fp8_linear does with its bias
 * argument (ops.py:345-346):
 *   fp8:  out = bf16( (a_fp8 . w_fp8^T) * scale_in * scale_w + bias )
 *   bf16: out = bf16( a_bf16 . w_bf16^T + bias )
 *   fp16: out = fp16( a_f16 . w_f16^T + bias )      (HDMOE_W_F16; bias fp16 or NULL) */
int hdmoe_linear_bias(int weight_dtype, const void* a, int rows, int K, int N, const void* w,
                      const float* scale_w_dev, const float* scale_in_dev, const void* bias_bf16,
                      void* out_bf16, hdmoe_stream_t stream);

/* Elementwise middle of model.py:238 for the unfused path: out = bf16(bf16(silu(a)) * b). */
int hdmoe_silu_mul_bf16(const void* a_bf16, const void* b_bf16, int64_t n, void* out_bf16,
                        hdmoe_stream_t stream);

/* F.gelu (erf form) of a bf16 tensor for the unfused Hunyuan3D expert, comfy/ldm/hunyuan3dv2_1/hunyuandit.py:14-26
 * (`gelu(proj(x))` when proj is not the plain bf16 Linear): out = bf16(gelu(fp32(x))). n % 8 == 0. */
int hdmoe_gelu_bf16(const void* x_bf16, int64_t n, void* out_bf16, hdmoe_stream_t stream);
/* the same on an fp16 tensor: out = fp16(gelu(fp32(x))) */
int hdmoe_gelu_f16(const void* x_f16, int64_t n, void* out_f16, hdmoe_stream_t stream);

/* `weight * scale_weight` or `input * scale_weight` of the scaled-fp8 Linear WITHOUT fp8
 * matmul (comfy/ops.py:407-410), after the operand was cast to bf16:
 *   out = bf16( bf16(src) * bf16(scale) ).   src: n elements of e4m3fn or bf16, n % 8 == 0. */
int hdmoe_scale_to_bf16(int src_dtype, const void* src, int64_t n, const float* scale_dev,
                        void* out_bf16, hdmoe_stream_t stream);

/* Weighted combine, model.py:319-324:
 *   out[t] = bf16( bf16( bf16(y[r0]*w[t,0]) + bf16(y[r1]*w[t,1]) ) + shared[t] ),  r_s = inv_perm[2t+s]
 * y_sorted [2T,D] bf16, topk_weight [T,2] bf16, shared [T,D] bf16 or NULL, out [T,D] bf16.
 * Deterministic (a gather, no atomics). D % 8 == 0. */
int hdmoe_combine(const void* y_sorted_bf16, const int32_t* inv_perm, const void* topk_weight_bf16,
                  const void* shared_bf16, int T, int D, void* out_bf16, hdmoe_stream_t stream);
/* The same combine with every tensor and every rounding in fp16: the weighted index_add_ in expert order plus the shared
 * expert of comfy/ldm/hunyuan3dv2_1/hunyuandit.py:176-187 at that dtype (a token meets at most two experts). */
int hdmoe_combine_f16(const void* y_sorted_f16, const int32_t* inv_perm, const void* topk_weight_f16,
                      const void* shared_f16, int T, int D, void* out_f16, hdmoe_stream_t stream);

/* Linear with bias (and optional erf GELU) over the expert row segments of a dispatched batch, plus optionally one
 * more group over all rows of another input (a shared expert), in one launch: the two stages of the GELU
 * feed-forward experts of comfy/ldm/hunyuan3dv2_1/hunyuandit.py:28-50 as MoEBlock (:114-188) runs them.
 *   out[r, :] = act( bf16( a[r, :] . W_e^T + bias_e ) ),  r in [offsets[e], offsets[e+1])
 * bf16 activations, weights [N,K] and biases [N] (bias NULL = none); K % 64 == 0, N % 256 == 0. */
#define HDMOE_ACT_NONE 0
#define HDMOE_ACT_GELU 1
typedef struct {
  const void* weight; /* [N,K] bf16 */
  const void* bias;   /* [N] bf16 or NULL */
} hdmoe_linear_weights;
int hdmoe_grouped_linear(const void* a_bf16, const int32_t* offsets, int rows_total, int E,
                         const hdmoe_linear_weights* experts, void* out_bf16, const void* a_static_bf16,
                         int rows_static, const hdmoe_linear_weights* shared, void* out_static_bf16, int K, int N,
                         int act, hdmoe_stream_t stream);
/* The same with fp16 activations, weights, biases and outputs (fp32 accumulation, one rounding to fp16 after the
 * bias, GELU of the rounded value rounded again). */
int hdmoe_grouped_linear_f16(const void* a_f16, const int32_t* offsets, int rows_total, int E,
                             const hdmoe_linear_weights* experts, void* out_f16, const void* a_static_f16,
                             int rows_static, const hdmoe_linear_weights* shared, void* out_static_f16, int K,
                             int N, int act, hdmoe_stream_t stream);

/* The same Linear as the first stage of a block, on the tokens themselves: expert e multiplies the rows its segment of
 * the dispatch holds, sorted row r being token perm[r] / 2 of x [T,K] (the rows `hidden_states[idx]` of
 * comfy/ldm/hunyuan3dv2_1/hunyuandit.py:176-186 select, read through the permutation instead of from a copy in
 * expert order), and the shared expert (NULL = none) all T rows. out [2T,N], out_shared [T,N]; act_dtype
 * HDMOE_W_BF16 or HDMOE_W_F16 is the element type of x, weights, biases and outputs. */
int hdmoe_grouped_linear_tokens(int act_dtype, const void* x, int T, const int32_t* perm, const int32_t* offsets, int E,
                                const hdmoe_linear_weights* experts, void* out, const hdmoe_linear_weights* shared,
                                void* out_shared, int K, int N, int act, hdmoe_stream_t stream);

/* Weight maintenance of a scaled-fp8 Linear (comfy/ops.py:419-426 set_weight, comfy/float.py:14-67):
 * out[i] = stochastic_round_e4m3fn( float16( src[i] / *scale_dev ) ), scale_dev NULL = 1. Each value lands on one of
 * its two e4m3fn neighbours, the upper one with probability equal to its position between them; |v| >= 448
 * saturates. The uniform numbers are Philox4x32-10(counter = i/4, key = seed), word i%4, not torch's generator:
 * same (src, scale, seed) -> same bytes, whatever the launch. src_dtype: HDMOE_SRC_F32 or HDMOE_SRC_BF16 (then the
 * scale and the quotient are rounded to bf16 first, as a bf16 tensor division does). out must be 4-byte aligned. */
#define HDMOE_SRC_BF16 0
#define HDMOE_SRC_F32 2
int hdmoe_stochastic_round_e4m3fn(int src_dtype, const void* src, int64_t n, const float* scale_dev, uint64_t seed,
                                  void* out_e4m3fn, hdmoe_stream_t stream);

/* Feed-forward branch of a HiDream block around the layer (comfy/ldm/hidream/model.py:429-433, 515-523):
 *   n   = LayerNorm(x, eps, no affine) * (1 + scale_mlp) + shift_mlp      -> hdmoe_ln_modulate_bf16
 *   out = gate_mlp * FFN(n) + x                                          -> hdmoe_combine_gated_residual
 * scale/shift/gate are [B, D] bf16 (one row per batch item; token t uses row t / tokens_per_batch); every
 * elementwise op rounds to bf16 as the reference's torch ops do. */
int hdmoe_ln_modulate_bf16(const void* x_bf16, const void* scale_bf16, const void* shift_bf16, int T, int D,
                           int tokens_per_batch, float eps, void* out_bf16, hdmoe_stream_t stream);
int hdmoe_combine_gated_residual(const void* y_sorted_bf16, const int32_t* inv_perm,
                                 const void* topk_weight_bf16, const void* shared_bf16,
                                 const void* gate_bf16, const void* residual_bf16, int tokens_per_batch,
                                 int T, int D, void* out_bf16, hdmoe_stream_t stream);

/* The same gate and residual behind a dense feed-forward (text stream, comfy/ldm/hidream/model.py:519-523):
 * out[t] = bf16( bf16(gate[t / tokens_per_batch] * y[t]) + residual[t] ). */
int hdmoe_gated_residual_bf16(const void* y_bf16, const void* gate_bf16, const void* residual_bf16,
                              int tokens_per_batch, int T, int D, void* out_bf16, hdmoe_stream_t stream);

/* ---- whole layer -------------------------------------------------------------- */

/* MOEFeedForwardSwiGLU.forward, model.py:307-325, as one call that enqueues
 * gate -> dispatch -> quantise/permute -> grouped gate/up GEMM with SiLU*mul ->
 * grouped down GEMM -> combine (+ shared expert through the same GEMMs). */
typedef struct hdmoe_layer_args {
  int T;            /* tokens (batch * sequence) */
  int D;            /* model width, 2560 for HiDream */
  int H;            /* routed expert hidden width */
  int Hs;           /* shared expert hidden width (0 = no shared expert) */
  int E;            /* routed experts */
  int weight_dtype; /* HDMOE_W_BF16 or HDMOE_W_E4M3FN */
  const void* x;            /* [T,D] bf16 device */
  const void* gate_w;       /* [E,D] bf16 device */
  const hdmoe_ffn_weights* experts; /* host array [E] */
  const hdmoe_ffn_weights* shared;  /* host pointer or NULL */
  void* out;                /* [T,D] bf16 device */
  void* workspace;          /* hdmoe_layer_workspace_bytes(...) bytes, 256-byte aligned, device */
  size_t workspace_bytes;
  /* optional device outputs (may be NULL): routing decision */
  int32_t* topk_idx;  /* [T,2] */
  void* topk_weight;  /* [T,2] bf16 */
  /* optional timing hook (may be NULL): HDMOE_NUM_STAGE_EVENTS hipEvent_t created by the caller.
   * Event i is recorded on `stream` before stage i and event i+1 after it; stages in order:
   * gate (with fp8 experts it also casts the activations), dispatch, permute (bf16 experts only), gate-up GEMM,
   * down GEMM, combine. NULL entries of the array are skipped (each recorded event costs a few microseconds
   * on the stream). */
  void** stage_events;
  /* optional block fusion (all three NULL = the plain layer). When set, x is the un-normalised token stream and
   * out = x + mod_gate * FFN( LayerNorm(x, ln_eps) * (1 + mod_scale) + mod_shift ); the normalised tokens live in
   * the workspace. [B, D] bf16 each, B = T / tokens_per_batch. */
  const void* mod_scale;
  const void* mod_shift;
  const void* mod_gate;
  int tokens_per_batch;
  float ln_eps;
  /* fp8 only. When w1/w3 of every routed expert and of the shared expert cast the tokens with the same factor, the
   * tokens are cast to e4m3fn once (one row per token instead of three) and every group of the gate/up GEMM reads
   * that copy. Whether they do is decided on the device, by the kernel that casts, from the values behind the
   * scale_in1 pointers at the time it runs (equal pointers and all-NULL are seen on the host). This field is a hint
   * of earlier versions and is not looked at. */
  int uniform_scale_in;
  /* Optional (may be NULL): one int32 the device can write (device memory, or pinned host memory through its device
   * address). w1 and w3 of a feed-forward read one cast of the tokens, so same_scale_in13 of hdmoe_ffn_weights is an
   * assertion about device values that the host may hold a stale copy of. The casting kernel verifies it: where the
   * two factors differ it writes NaN rows (the output of the call is then NaN, not a wrong number) and sets this
   * word to 1. A caller that caches its comparison of the values can poll the word and drop the cache. */
  int32_t* scale_check;
  /* With a few hundred to about two thousand tokens the down projection is cut along K, and which of the candidate
   * cuts runs is chosen on the device from the experts' segment sizes (the cut that fills one round of blocks). The
   * fp32 summation order of a row then depends on how the OTHER tokens of the batch were routed: the same token can
   * differ in the last bit of its output between two batches. Nonzero here fixes the cut from the sizes alone (the
   * cost model's choice), which makes every row's bytes a function of that row, its expert's weights and T only, at
   * 2 to 10 % of the layer's time at those sizes. */
  int fixed_k_cut;
} hdmoe_layer_args;

#define HDMOE_NUM_STAGES 6
#define HDMOE_NUM_STAGE_EVENTS (HDMOE_NUM_STAGES + 1)

/* The workspace size already includes room for the normalised tokens of the block fusion. */
size_t hdmoe_layer_workspace_bytes(int T, int D, int H, int Hs, int E, int weight_dtype);
int hdmoe_moe_ffn(const hdmoe_layer_args* args, hdmoe_stream_t stream);

/* FeedForwardSwiGLU.forward, model.py:237-238, for one dense FFN (the shared expert on its own, the text-token
 * feed-forward, or a block built with num_routed_experts == 0): out = w2( silu(w1 x) * w3 x ) with the same
 * per-Linear semantics as above. x [rows,D] bf16 -> out [rows,D] bf16. Three launches (fp8: quantise, gate/up GEMM
 * with the SiLU*mul epilogue, down GEMM; bf16: the two GEMMs). workspace: hdmoe_ffn_workspace_bytes(...) bytes,
 * 256-byte aligned, device. */
size_t hdmoe_ffn_workspace_bytes(int rows, int D, int H, int weight_dtype);
int hdmoe_ffn_swiglu(int weight_dtype, const void* x_bf16, int rows, int D, int H,
                     const hdmoe_ffn_weights* w, void* out_bf16, void* workspace,
                     size_t workspace_bytes, hdmoe_stream_t stream);

/* Where the pieces of the workspace live, for tests that inspect intermediates. */
typedef struct hdmoe_layer_layout {
  size_t topk_idx, topk_weight, counts, offsets, perm, inv_perm, dispatch_ws;
  size_t a, h, y, normed, partials, flags, total;
} hdmoe_layer_layout;
int hdmoe_layer_layout_get(int T, int D, int H, int Hs, int E, int weight_dtype,
                           hdmoe_layer_layout* out);

#ifdef __cplusplus
}
#endif
#endif /* HDMOE_H */
