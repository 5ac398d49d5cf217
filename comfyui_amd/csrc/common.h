// Host-side helpers shared by the translation units of libhdmoe.
#pragma once
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include "../../include/hdmoe.h"

// thread-local message behind hdmoe_last_error()
char* hdmoe_error_buffer();
constexpr int HDMOE_ERRBUF = 512;

static inline int hdmoe_fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(hdmoe_error_buffer(), HDMOE_ERRBUF, fmt, ap);
  va_end(ap);
  return code;
}

// Launch errors are read with hipGetLastError only: it does not synchronise.
static inline int hdmoe_check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return hdmoe_fail(HDMOE_E_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return HDMOE_OK;
}

#define HDMOE_REQUIRE_PTR(p)                                                   \
  do {                                                                         \
    if ((p) == nullptr) return hdmoe_fail(HDMOE_E_NULL, "%s: %s is NULL", __func__, #p); \
  } while (0)

// w1 and w3 of a SwiGLU feed-forward quantise the same input once, with scale_in1 (see hdmoe_ffn_weights).
static inline int hdmoe_check_scale_in13(const char* what, const hdmoe_ffn_weights& w, int index) {
  if (w.scale_in1 == w.scale_in3) return HDMOE_OK;
  if (w.scale_in1 == nullptr || w.scale_in3 == nullptr)
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: group %d: w1 and w3 disagree on having a scale_input", what, index);
  if (!w.same_scale_in13)
    return hdmoe_fail(HDMOE_E_SHAPE,
                      "%s: group %d: scale_in1 and scale_in3 are different pointers and same_scale_in13 is not set "
                      "(the fused kernels quantise the input once, so the two values must be equal)", what, index);
  return HDMOE_OK;
}

static inline size_t hdmoe_align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

// gate kernels: which kernel casts (with_cast: fp8 experts; with_ln: LayerNorm + modulation inside the kernel), its
// tokens per block (a pure function of the sizes) and the bytes of the per-block expert histograms
int hdmoe_gate_tokens_per_block(int T, int D, int E, bool with_cast, bool with_ln);
size_t hdmoe_gate_hist_bytes(int T, int D, int E, bool with_cast);

// Few rows per segment: one m-tile per group and the experts' 256-token tiles half empty on average (up to 256 tokens
// in a top-2 layer of 4 experts). Such launches run in the forms of the GEMM kernels that skip padding, and their down
// projection is cut along K for 128-token tiles. One rule for the launcher and for the K cut (which depends on the
// sizes only, never on the form switches, so that every form of a kernel adds up the same parts in the same order).
static inline bool hdmoe_few_rows(int rows_dyn, int n_dyn, int rows_static) {
  return (n_dyn <= 0 || rows_dyn <= 128 * n_dyn) && rows_static <= 256;
}

// What the gate + cast kernel of the one-call layer decides and verifies from the values behind the scale pointers
// (see GateQuant in gate.hip).
struct HdmoeGateScaleChecks {
  bool decide;               // the kernel picks one row per token or a row per slot and reports it in *layout_flag
  bool with_shared;          // row-per-slot layout: also write the shared expert's token-order copy
  int32_t* layout_flag;      // device word: 1 = one row per token
  int32_t* scale_check;      // optional word (device, or host memory the device can write): set to 1 on a mismatch
  const float* scale_in3[HDMOE_MAX_EXPERTS];  // scale_input of every expert's w3
  const float* shared_scale3;                 // of the w3 the shared_scale passed beside this belongs to
};

// A second description of the gathered token operand of a grouped GEMM, taken when *flag reads 0 on the device.
struct HdmoeAltOperand {
  const int32_t* flag;
  const uint8_t* a;
  int rows;      // rows of a
  int shift;     // row = gather[r] >> shift
};

constexpr int HDMOE_NUM_CU = 256;   // MI355X
constexpr int HDMOE_NUM_XCD = 8;

// ---- K cuts of a down projection (split K) ---------------------------------------------------------------------
// The host does not know the routing, and whether a cut pays depends on how many tiles the experts' segments really
// make: a cut whose tiles fit one round of blocks beats every other, one tile more and it needs a second round. So the
// host lists candidate cuts (most parts first, each expected to fit under favourable routing) and a last entry that is
// taken when none fits; the GEMM kernel and the kernel that adds the parts up both evaluate hdmoe_plan_pick on the
// segment bounds the dispatch left on the device, and so agree without the host ever seeing them.
constexpr int HDMOE_PLAN_MAX = 12;
struct HdmoeSplitPlan {
  int n;                     // entries in use; 1 = a fixed cut
  int pd[HDMOE_PLAN_MAX];    // K parts of a tile of the experts' groups
  int ps[HDMOE_PLAN_MAX];    // K parts of a tile of the static group (the shared expert)
  int bm;                    // tile height (tokens) the launch runs with
  int max_tiles;             // an entry before the last is taken only if its tiles number at most this
};

// mt_dyn / mt_static: m-tiles (tile height plan.bm) of all experts' segments / of the static group; ntiles_n: tiles
// along the output features. Returns the index of the entry to run.
__host__ __device__ inline int hdmoe_plan_pick(const HdmoeSplitPlan& plan, int mt_dyn, int mt_static, int ntiles_n) {
  for (int i = 0; i + 1 < plan.n; ++i)
    if ((mt_dyn * plan.pd[i] + mt_static * plan.ps[i]) * ntiles_n <= plan.max_tiles) return i;
  return plan.n - 1;
}

