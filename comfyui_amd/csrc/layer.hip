// Whole-layer entry point: enqueues every stage of MOEFeedForwardSwiGLU.forward
// (/root/reference/comfy/ldm/hidream/model.py:307-325) on one stream, with all
// intermediates in a caller-provided workspace. Also hosts the library-wide pieces
// (version, thread-local error text).
#include "common.h"

int hdmoe_launch_ffn_gemm(bool swiglu, int weight_dtype, const uint8_t* a_dyn, const int32_t* offsets, int rows_dyn,
                          int n_dyn, const hdmoe_ffn_weights* experts, uint8_t* out_dyn, const uint8_t* a_static,
                          int rows_static, const hdmoe_ffn_weights* shared, uint8_t* out_static, int K_dyn, int N_dyn,
                          int K_static, int N_static, hipStream_t s, const char* what,
                          const int32_t* gather_dyn = nullptr, int gather_rows = 0, float* partial = nullptr,
                          int nparts = 1, int gather_shift = 0, bool reduce = true,
                          const HdmoeSplitPlan* plan = nullptr, const HdmoeAltOperand* alt = nullptr);
int hdmoe_launch_combine_partials(const float* partial, long long part_stride, const HdmoeSplitPlan& plan,
                                  int rows_dyn, int n_dyn,
                                  const int32_t* offsets, bool fp8, const hdmoe_ffn_weights* experts,
                                  const hdmoe_ffn_weights* shared, const int32_t* inv_perm, const void* topk_weight_bf16,
                                  const void* gate_bf16, const void* residual_bf16, int tokens_per_batch, int T, int D,
                                  void* out_bf16, hipStream_t s, const char* what);
int hdmoe_down_parts(int rows_dyn, int n_dyn, int rows_static, int N, int K_dyn, int K_static, int weight_dtype,
                     HdmoeSplitPlan* plan = nullptr);
int hdmoe_check_gemm_shape(const char* what, int weight_dtype, long rows, int K, int N, int feat_per_tile);
int hdmoe_launch_quant_dispatch(const void* x_bf16, const int32_t* perm, const int32_t* offsets, int T, int D, int E,
                                const float* const* scale_input, const float* shared_scale, bool with_shared,
                                void* a_fp8, hipStream_t s, const char* what);
int hdmoe_launch_gate_quant(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E, int32_t* topk_idx,
                            void* topk_weight_bf16, const float* const* scale_input, const float* shared_scale,
                            void* xq_routed, void* xq_shared, hipStream_t s, const char* what,
                            const void* mod_scale = nullptr, const void* mod_shift = nullptr, int tokens_per_batch = 0,
                            float ln_eps = 0.0f, int32_t* block_hist = nullptr,
                            const HdmoeGateScaleChecks* checks = nullptr);
int hdmoe_launch_gate(const void* x_bf16, const void* gate_w_bf16, int T, int D, int E, int32_t* topk_idx,
                      void* topk_weight_bf16, int32_t* block_hist, hipStream_t s, const char* what);
int hdmoe_launch_dispatch_scatter(const int32_t* topk_idx, int T, int E, int32_t* counts, int32_t* offsets,
                                  int32_t* perm, int32_t* inv_perm, const int32_t* block_hist, int tokens_per_hist,
                                  hipStream_t s, const char* what);
bool hdmoe_gate_quant_takes_ln(int D, int E);
int hdmoe_launch_quant_rows(const void* x_bf16, int64_t rows, int D, const float* scale_input_dev,
                            const float* scale_input_also_dev, void* out_fp8, hipStream_t s, const char* what);
int hdmoe_launch_combine(const void* y_sorted_bf16, const int32_t* inv_perm, const void* topk_weight_bf16,
                         const void* shared_bf16, const void* gate_bf16, const void* residual_bf16, int tokens_per_batch,
                         int T, int D, void* out_bf16, hipStream_t s, const char* what, bool f16 = false);

char* hdmoe_error_buffer() {
  static thread_local char buf[HDMOE_ERRBUF] = {0};
  return buf;
}

extern "C" int hdmoe_version(void) { return HDMOE_VERSION; }
extern "C" const char* hdmoe_last_error(void) { return hdmoe_error_buffer(); }

extern "C" int hdmoe_layer_layout_get(int T, int D, int H, int Hs, int E, int weight_dtype,
                                      hdmoe_layer_layout* out) {
  HDMOE_REQUIRE_PTR(out);
  if (T < 0 || D <= 0 || H <= 0 || Hs < 0 || E < 1 || E > HDMOE_MAX_EXPERTS ||
      (weight_dtype != HDMOE_W_BF16 && weight_dtype != HDMOE_W_E4M3FN))
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_layer_layout_get: T=%d D=%d H=%d Hs=%d E=%d dtype=%d", T, D, H, Hs, E,
                      weight_dtype);
  const size_t eb = weight_dtype == HDMOE_W_E4M3FN ? 1 : 2;
  const size_t n = (size_t)T * HDMOE_TOPK;
  const bool fp8 = weight_dtype == HDMOE_W_E4M3FN;
  size_t off = 0;
  auto take = [&](size_t bytes) { size_t o = off; off = hdmoe_align_up(off + bytes, 256); return o; };
  out->topk_idx = take(n * 4);
  out->topk_weight = take(n * 2);
  out->counts = take((size_t)E * 4);
  out->offsets = take((size_t)(E + 1) * 4);
  out->perm = take(n * 4);
  out->inv_perm = take(n * 4);
  // per-block expert histograms of the gate kernel (the first pass of the dispatch); large enough for hdmoe_dispatch
  // too, for a caller that composes the layer from the stages inside this workspace
  {
    const size_t a = hdmoe_gate_hist_bytes(T, D, E, fp8), b = hdmoe_dispatch_workspace_bytes(T, E);
    out->dispatch_ws = take(a > b ? a : b);
  }
  // a (fp8 only; bf16 weights multiply the tokens themselves): the tokens' e4m3fn rows per flat slot [2T,D], then
  // the token-order copy for the shared expert [T,D]
  out->a = take(fp8 ? (n + (Hs > 0 ? (size_t)T : 0)) * D * eb : 0);
  // h: routed [2T,H] then shared [T,Hs]
  out->h = take((n * H + (size_t)T * Hs) * eb);
  // y: routed [2T,D] then shared [T,D], bf16
  out->y = take((n + (Hs > 0 ? (size_t)T : 0)) * D * 2);
  // normalised + modulated tokens of the optional block fusion, [T,D] bf16
  out->normed = take((size_t)T * D * 2);
  // fp32 partial sums of a down projection cut along K (small token counts), [parts][2T + T][D]
  const int parts = hdmoe_down_parts((int)n, E, Hs > 0 ? T : 0, D, H, Hs, weight_dtype);
  out->partials = take(parts > 1 ? (size_t)parts * (n + (Hs > 0 ? (size_t)T : 0)) * D * 4 : 0);
  // one word the gate + cast kernel leaves for the gate/up GEMM: which layout of the fp8 tokens it wrote
  out->flags = take(256);
  out->total = off;
  return HDMOE_OK;
}

extern "C" size_t hdmoe_layer_workspace_bytes(int T, int D, int H, int Hs, int E, int weight_dtype) {
  hdmoe_layer_layout l;
  if (hdmoe_layer_layout_get(T, D, H, Hs, E, weight_dtype, &l) != HDMOE_OK) return 0;
  return l.total;
}

extern "C" int hdmoe_moe_ffn(const hdmoe_layer_args* p, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(p);
  HDMOE_REQUIRE_PTR(p->x);
  HDMOE_REQUIRE_PTR(p->gate_w);
  HDMOE_REQUIRE_PTR(p->experts);
  HDMOE_REQUIRE_PTR(p->out);
  HDMOE_REQUIRE_PTR(p->workspace);
  const int T = p->T, D = p->D, H = p->H, Hs = p->Hs, E = p->E, wd = p->weight_dtype;
  hdmoe_layer_layout l;
  if (int rc = hdmoe_layer_layout_get(T, D, H, Hs, E, wd, &l)) return rc;
  if (Hs > 0) HDMOE_REQUIRE_PTR(p->shared);
  if (p->workspace_bytes < l.total || (reinterpret_cast<uintptr_t>(p->workspace) & 255))
    return hdmoe_fail(HDMOE_E_WORKSPACE, "hdmoe_moe_ffn: workspace %zu bytes, need %zu (256-byte aligned)",
                      p->workspace_bytes, l.total);
  const long n = (long)T * HDMOE_TOPK;
  if (int rc = hdmoe_check_gemm_shape("hdmoe_moe_ffn (gate/up)", wd, n + T, D, H, 128)) return rc;
  if (int rc = hdmoe_check_gemm_shape("hdmoe_moe_ffn (down)", wd, n, H, D, 256)) return rc;
  if (Hs > 0) {
    if (int rc = hdmoe_check_gemm_shape("hdmoe_moe_ffn (shared gate/up)", wd, T, D, Hs, 128)) return rc;
    if (int rc = hdmoe_check_gemm_shape("hdmoe_moe_ffn (shared down)", wd, T, Hs, D, 256)) return rc;
  }
  const bool fused_block = p->mod_scale != nullptr || p->mod_shift != nullptr || p->mod_gate != nullptr;
  if (fused_block) {
    HDMOE_REQUIRE_PTR(p->mod_scale);
    HDMOE_REQUIRE_PTR(p->mod_shift);
    HDMOE_REQUIRE_PTR(p->mod_gate);
    if (p->tokens_per_batch <= 0 || T % p->tokens_per_batch != 0)
      return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_moe_ffn: tokens_per_batch=%d does not divide T=%d", p->tokens_per_batch, T);
  }
  if (T == 0) return HDMOE_OK;

  const bool fp8 = wd == HDMOE_W_E4M3FN;
  const size_t eb = fp8 ? 1 : 2;
  uint8_t* ws = static_cast<uint8_t*>(p->workspace);
  int32_t* idx = p->topk_idx ? p->topk_idx : reinterpret_cast<int32_t*>(ws + l.topk_idx);
  void* tw = p->topk_weight ? p->topk_weight : static_cast<void*>(ws + l.topk_weight);
  int32_t* counts = reinterpret_cast<int32_t*>(ws + l.counts);
  int32_t* offsets = reinterpret_cast<int32_t*>(ws + l.offsets);
  int32_t* perm = reinterpret_cast<int32_t*>(ws + l.perm);
  int32_t* inv_perm = reinterpret_cast<int32_t*>(ws + l.inv_perm);
  // The gate kernel also counts (one expert histogram per block of tokens), so the dispatch is its scatter pass alone.
  int32_t* const hist = reinterpret_cast<int32_t*>(ws + l.dispatch_ws);
  uint8_t* a_routed = ws + l.a;
  uint8_t* a_shared = a_routed + (size_t)n * D * eb;  // fp8 only
  uint8_t* h_routed = ws + l.h;
  uint8_t* h_shared = h_routed + (size_t)n * H * eb;
  uint8_t* y_routed = ws + l.y;
  uint8_t* y_shared = y_routed + (size_t)n * D * 2;
  hipStream_t s = static_cast<hipStream_t>(stream);

  if (fp8) {
    for (int e = 0; e < E; ++e)
      if (int rc = hdmoe_check_scale_in13("hdmoe_moe_ffn", p->experts[e], e)) return rc;
    if (Hs > 0)
      if (int rc = hdmoe_check_scale_in13("hdmoe_moe_ffn (shared expert)", *p->shared, E)) return rc;
  }

  int ev = 0;
  hipError_t ev_err = hipSuccess;
  auto mark = [&]() {
    if (p->stage_events && p->stage_events[ev] != nullptr) {
      const hipError_t e = hipEventRecord(static_cast<hipEvent_t>(p->stage_events[ev]), s);
      if (e != hipSuccess && ev_err == hipSuccess) ev_err = e;
    }
    ++ev;
  };
  // the tokens the feed-forward sees: x itself, or LayerNorm(x) * (1 + scale) + shift (timed with the gate stage)
  const void* xin = p->x;
  mark();
  // fp8 experts at the register kernel's shape: LayerNorm + modulation happen inside the gate + cast kernel and
  // the normalised tokens are never written as bf16
  const bool ln_in_gate = fused_block && fp8 && hdmoe_gate_quant_takes_ln(D, E);
  if (fused_block && !ln_in_gate) {
    void* normed = ws + l.normed;
    if (int rc = hdmoe_ln_modulate_bf16(p->x, p->mod_scale, p->mod_shift, T, D, p->tokens_per_batch, p->ln_eps, normed,
                                        stream))
      return rc;
    xin = normed;
  }
  // fp8 experts: the gate kernel also casts each token to e4m3fn while it holds the row. When every Linear that reads
  // the tokens (w1/w3 of every routed expert and of the shared expert) has the same scale_input, one row per token
  // serves them all and the gate/up GEMM reads row perm[r] / 2 of it. Otherwise the token is cast for its two experts
  // (rows 2t, 2t+1 of a_routed, i.e. in flat slot order) and for the shared expert, and the GEMM reads the routed rows
  // through the permutation instead of from a permuted copy.
  // Which of the two it is depends on the VALUES of the scale_inputs. The host sees pointers: all the same pointer
  // (all NULL included) is one copy, a mix of NULL (clamp rule) and non-NULL is never one copy; for different non-NULL
  // pointers the gate kernel compares the values on the device, writes the layout that fits and leaves a flag the
  // gate/up GEMM reads (uniform_scale_in of the arguments is not needed for that and is not looked at). The same
  // kernel checks that w1 and w3 of every group cast the tokens alike (they read one cast).
  bool one_copy = false, decide = false;
  if (fp8) {
    const float* first = p->experts[0].scale_in1;
    bool same_ptr = true, mixed = false;
    for (int e = 0; e < E; ++e) {
      same_ptr = same_ptr && p->experts[e].scale_in1 == first;
      mixed = mixed || ((p->experts[e].scale_in1 == nullptr) != (first == nullptr));
    }
    if (Hs > 0) {
      same_ptr = same_ptr && p->shared->scale_in1 == first;
      mixed = mixed || ((p->shared->scale_in1 == nullptr) != (first == nullptr));
    }
    one_copy = same_ptr;
    decide = !same_ptr && !mixed;
  }
  int32_t* const layout_flag = reinterpret_cast<int32_t*>(ws + l.flags);
  if (fp8) {
    const float* sin[HDMOE_MAX_EXPERTS];
    HdmoeGateScaleChecks checks = {};
    for (int e = 0; e < E; ++e) {
      sin[e] = p->experts[e].scale_in1;
      checks.scale_in3[e] = p->experts[e].scale_in3;
    }
    // the scale of the token-order copy: the shared expert's, or (one copy for all, no shared expert) the experts'
    const hdmoe_ffn_weights& token_w = Hs > 0 ? *p->shared : p->experts[0];
    checks.decide = decide;
    checks.with_shared = Hs > 0;
    checks.layout_flag = layout_flag;
    checks.scale_check = p->scale_check;
    // the one copy sits where the shared expert's copy would (without a shared expert that room does not exist: the
    // start of the routed rows' room then; only one of the two layouts is written in a call)
    if (Hs == 0) a_shared = a_routed;
    const bool token_copy = Hs > 0 || one_copy || decide;
    checks.shared_scale3 = token_copy ? token_w.scale_in3 : nullptr;
    if (int rc = hdmoe_launch_gate_quant(xin, p->gate_w, T, D, E, idx, tw, sin, token_copy ? token_w.scale_in1 : nullptr,
                                         one_copy ? nullptr : a_routed, token_copy ? a_shared : nullptr, s,
                                         "hdmoe_moe_ffn (gate + quantise)",
                                         ln_in_gate ? p->mod_scale : nullptr, ln_in_gate ? p->mod_shift : nullptr,
                                         p->tokens_per_batch, p->ln_eps, hist, &checks))
      return rc;
  } else {
    if (D % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_moe_ffn: D=%d must be a multiple of 8", D);
    if (int rc = hdmoe_launch_gate(xin, p->gate_w, T, D, E, idx, tw, hist, s, "hdmoe_moe_ffn (gate)")) return rc;
  }
  mark();
  if (int rc = hdmoe_launch_dispatch_scatter(idx, T, E, counts, offsets, perm, inv_perm, hist,
                                             hdmoe_gate_tokens_per_block(T, D, E, fp8, ln_in_gate), s, "hdmoe_moe_ffn (dispatch)"))
    return rc;
  mark();

  // bf16 weights: the GEMM reads the tokens themselves, the routed rows through the permutation (row perm[r] / 2
  // of x), so no permuted copy is written
  const uint8_t* a_static = nullptr;
  if (fp8) {
    if (Hs > 0) a_static = a_shared;
  } else {
    a_static = static_cast<const uint8_t*>(xin);
  }

  mark();
  // gate/up projections + SiLU*mul, routed experts and shared expert in one launch
  // the routed operand holds one row per token (else one per flat slot); when the gate kernel decided, the
  // one-row-per-token form is described here and the other one as the alternative its flag selects
  const bool per_token = one_copy || decide || !fp8;
  const uint8_t* const a_dyn = !fp8 ? static_cast<const uint8_t*>(xin) : (per_token ? a_shared : a_routed);
  HdmoeAltOperand alt;
  alt.flag = layout_flag;
  alt.a = a_routed;
  alt.rows = (int)n;
  alt.shift = 0;
  if (int rc = hdmoe_launch_ffn_gemm(true, wd, a_dyn, offsets, (int)n, E, p->experts, h_routed,
                                     a_static, Hs > 0 ? T : 0, p->shared, h_shared, D, H, D, Hs, s,
                                     "hdmoe_moe_ffn (gate/up)", perm, per_token ? T : (int)n, nullptr, 1,
                                     per_token ? 1 : 0, true, nullptr, decide ? &alt : nullptr))
    return rc;
  mark();
  // down projections, both in one launch
  HdmoeSplitPlan plan;  // candidate cuts; the kernels pick one by the real segment sizes
  const int parts = hdmoe_down_parts((int)n, E, Hs > 0 ? T : 0, D, H, Hs, wd, &plan);
  if (p->fixed_k_cut != 0 && plan.n > 1) {  // the cost model's entry, whatever the routing
    plan.pd[0] = plan.pd[plan.n - 1];
    plan.ps[0] = plan.ps[plan.n - 1];
    plan.n = 1;
  }
  if (int rc = hdmoe_launch_ffn_gemm(false, wd, h_routed, offsets, (int)n, E, p->experts, y_routed, h_shared,
                                     Hs > 0 ? T : 0, p->shared, y_shared, H, D, Hs, D, s, "hdmoe_moe_ffn (down)",
                                     nullptr, 0, parts > 1 ? reinterpret_cast<float*>(ws + l.partials) : nullptr, parts,
                                     0, /*reduce=*/false, &plan))
    return rc;
  mark();
  // cut along K: the combine adds the parts up itself (no launch and no bf16 copy of the rows in between)
  const int rc = parts > 1
      ? hdmoe_launch_combine_partials(reinterpret_cast<const float*>(ws + l.partials),
                                      (long long)(n + (Hs > 0 ? (size_t)T : 0)) * D, plan, (int)n, E, offsets, fp8,
                                      p->experts, Hs > 0 ? p->shared : nullptr, inv_perm, tw,
                                      fused_block ? p->mod_gate : nullptr, fused_block ? p->x : nullptr,
                                      fused_block ? p->tokens_per_batch : 1, T, D, p->out, s, "hdmoe_moe_ffn (combine)")
      : hdmoe_launch_combine(y_routed, inv_perm, tw, Hs > 0 ? y_shared : nullptr,
                             fused_block ? p->mod_gate : nullptr, fused_block ? p->x : nullptr,
                             fused_block ? p->tokens_per_batch : 1, T, D, p->out, s, "hdmoe_moe_ffn (combine)");
  mark();
  if (rc == HDMOE_OK && ev_err != hipSuccess)
    return hdmoe_fail(HDMOE_E_LAUNCH, "hdmoe_moe_ffn: hipEventRecord on a stage event: %s", hipGetErrorString(ev_err));
  return rc;
}

extern "C" size_t hdmoe_ffn_workspace_bytes(int rows, int D, int H, int weight_dtype) {
  if (rows < 0 || D <= 0 || H <= 0 || (weight_dtype != HDMOE_W_BF16 && weight_dtype != HDMOE_W_E4M3FN)) return 0;
  const size_t eb = weight_dtype == HDMOE_W_E4M3FN ? 1 : 2;
  // fp8: quantised copy of x, then h; bf16: h only (x itself is the GEMM operand); then the fp32 partial sums of a
  // down projection cut along K (few rows)
  const size_t a = weight_dtype == HDMOE_W_E4M3FN ? hdmoe_align_up((size_t)rows * D * eb, 256) : 0;
  const int parts = hdmoe_down_parts(0, 0, rows, D, 0, H, weight_dtype);
  const size_t pbytes = parts > 1 ? hdmoe_align_up((size_t)parts * rows * D * 4, 256) : 0;
  return a + hdmoe_align_up((size_t)rows * H * eb, 256) + pbytes;
}

extern "C" int hdmoe_ffn_swiglu(int weight_dtype, const void* x_bf16, int rows, int D, int H,
                                const hdmoe_ffn_weights* w, void* out_bf16, void* workspace, size_t workspace_bytes,
                                hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(x_bf16);
  HDMOE_REQUIRE_PTR(w);
  HDMOE_REQUIRE_PTR(out_bf16);
  HDMOE_REQUIRE_PTR(workspace);
  if (int rc = hdmoe_check_gemm_shape("hdmoe_ffn_swiglu (gate/up)", weight_dtype, rows, D, H, 128)) return rc;
  if (int rc = hdmoe_check_gemm_shape("hdmoe_ffn_swiglu (down)", weight_dtype, rows, H, D, 256)) return rc;
  const size_t need = hdmoe_ffn_workspace_bytes(rows, D, H, weight_dtype);
  if (workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255))
    return hdmoe_fail(HDMOE_E_WORKSPACE, "hdmoe_ffn_swiglu: workspace %zu bytes, need %zu (256-byte aligned)",
                      workspace_bytes, need);
  if (rows == 0) return HDMOE_OK;
  const bool fp8 = weight_dtype == HDMOE_W_E4M3FN;
  if (fp8)
    if (int rc = hdmoe_check_scale_in13("hdmoe_ffn_swiglu", *w, 0)) return rc;
  hipStream_t s = static_cast<hipStream_t>(stream);
  uint8_t* ws = static_cast<uint8_t*>(workspace);
  const uint8_t* a = static_cast<const uint8_t*>(x_bf16);
  uint8_t* h = ws;
  if (fp8) {
    if (D % 8 != 0) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_ffn_swiglu: D=%d must be a multiple of 8", D);
    // one cast for w1 and w3, made with w1's factor and checked against w3's on the device
    if (int rc = hdmoe_launch_quant_rows(x_bf16, rows, D, w->scale_in1, w->scale_in3, ws, s, "hdmoe_ffn_swiglu (quantise)"))
      return rc;
    a = ws;
    h = ws + hdmoe_align_up((size_t)rows * D, 256);
  }
  if (int rc = hdmoe_launch_ffn_gemm(true, weight_dtype, nullptr, nullptr, 0, 0, nullptr, nullptr, a, rows, w, h, 0, 0, D, H,
                                     s, "hdmoe_ffn_swiglu (gate/up)"))
    return rc;
  const int parts = hdmoe_down_parts(0, 0, rows, D, 0, H, weight_dtype);
  float* partial = parts > 1 ? reinterpret_cast<float*>(h + hdmoe_align_up((size_t)rows * H * (fp8 ? 1 : 2), 256)) : nullptr;
  return hdmoe_launch_ffn_gemm(false, weight_dtype, nullptr, nullptr, 0, 0, nullptr, nullptr, h, rows, w,
                               static_cast<uint8_t*>(out_bf16), 0, 0, H, D, s, "hdmoe_ffn_swiglu (down)", nullptr, 0,
                               partial, parts);
}
