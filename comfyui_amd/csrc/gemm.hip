// Grouped "NT" GEMM on the gfx950 matrix cores for the expert feed-forwards:
//   out[r, n] = epilogue( sum_k a[r, k] * w_g[n, k] ),  r in the row segment of group g.
// Replaces the per-expert operations.Linear calls of FeedForwardSwiGLU.forward
// (/root/reference/comfy/ldm/hidream/model.py:237-238) as fp8_linear evaluates them
// (/root/reference/comfy/ops.py:345-348: fp8 x fp8 products, fp32 accumulation,
// * scale_input*scale_weight, rounded to bf16) or, for bf16 weights, as a bf16
// Linear does (ops.py:107-115).
//
// Both operands are K-contiguous, which is the layout the MFMA wants: a lane feeds
// 32 (fp8) or 16 (bf16) consecutive K bytes of one row. Weights take the MFMA "A"
// slot (rows of the 32x32 result = output features) and tokens the "B" slot (columns
// = tokens), so a lane ends up with 4 consecutive features of one token per
// accumulator quad; the packed quads are transposed through LDS and leave as
// 128-byte row pieces.
//
// Block = 512 threads = 8 waves (2 per SIMD), block tile 256 tokens x 256 weight rows,
// K step 128 bytes, 2 LDS stages of 64 KiB filled by buffer_load ... lds (global ->
// LDS without passing through registers). Wave (wq, wt) owns weight rows {wq*32..+32}
// of each 128-row half and tokens {wt*128..+128}: 2x4 MFMA tiles of 32x32, 128 fp32
// accumulators per lane. In SwiGLU mode the two 128-row halves of the weight tile are
// the SAME 128 hidden features of w1 (gate) and w3 (up), so silu(gate)*up is formed
// in registers and the [rows, 2H] intermediate never exists.
//
// LDS tile layout: row-major, 128 bytes per row, 16-byte chunks XOR-swizzled with
// f(row) = ((row>>1)&7) ^ ((row&1)<<2) so that the 16-byte MFMA fragment reads of 8
// or 16 consecutive rows hit distinct banks. The global->LDS path writes LDS linearly
// per lane, so the swizzle is applied to the global address each lane fetches.
//
// Groups: row segments come from the dispatch offsets on the device (no host sync).
// The grid is sized for the worst case; a block first decodes (group, m-tile, n-tile)
// from its index and exits if its index is past the real tile count. Block ids are
// remapped so that each XCD (ids congruent mod 8) walks a contiguous range of tiles,
// 4 m-tiles deep, and its L2 sees each operand tile reused by neighbouring blocks.
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "common.h"
#include "numfmt.h"

namespace {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

constexpr int BN = 256;        // weight rows per block tile
constexpr int BK = 128;        // K bytes per stage
constexpr int STAGES = 2;
// Tokens per block tile: 2 wave rows x TT MFMA tiles of 32 tokens. TT = 4 (256 tokens) everywhere; the fp8 kernels
// also exist with TT = 5 (320 tokens: 10 % fewer operand bytes per MAC and fewer tiles), which the launcher picks
// when its tile count fills the chip as well.
constexpr int MAX_SLABS = 5;  // 64-row slabs of the largest token tile (arrays of dependent size in lambda
                              // signatures make the host pass drop the kernel stubs)
template <int TT>
struct TileCfg {
  static constexpr int BM = 64 * TT;                      // tokens per block tile
  // dynamic LDS of a block; the 128-token tile (TT = 2) has room for a third stage
  static constexpr int SMEM = (TT == 2 ? 3 : STAGES) * (BM + 256) * 128;
};
constexpr int GROUP_M = 4;     // m-tiles per raster band
constexpr int NTHREADS = 512;
constexpr int MAX_GROUPS = HDMOE_MAX_EXPERTS + 1;

// F16_PLAIN_BIAS: fp16 activations, weights, bias and outputs (the dtype the Hunyuan3D block runs in where the device
// takes it); the bf16 kernel with the other 16-bit MFMA and the other rounding.
enum Mode { FP8_SWIGLU = 0, FP8_PLAIN = 1, BF16_SWIGLU = 2, BF16_PLAIN = 3, BF16_PLAIN_BIAS = 4, FP8_PLAIN_BIAS = 5,
            F16_PLAIN_BIAS = 6 };

struct GemmGroup {
  const uint8_t* a;     // activations; row indices below are relative to this base
  const int32_t* gather;  // NULL: row r of the group is row r of a; else it is row gather[r] >> gather_shift of a (a_rows rows)
  int gather_shift;       // 1: gather holds flat slots 2t+s and a has one row per token
  int a_rows;
  const uint8_t* b0;    // plain: W [N,K]; swiglu: w1 [H,K]
  const uint8_t* b1;    // swiglu: w3 [H,K]
  const float* sb0;     // scale_weight of b0 (fp8)
  const float* sb1;     // scale_weight of b1 (fp8, swiglu)
  const float* s_in;    // scale_input of this Linear (fp8), NULL = 1
  const float* s_in_b;  // swiglu: scale_input of the w3 Linear (its value may differ from w1's where both round to the
                        // same cast factor); NULL = s_in
  const float* s_next;  // scale_input of the Linear that consumes the output (fp8 swiglu), NULL = clamp rule
  uint8_t* out;         // [rows, n_out] in the element type of the mode
  int row_begin;        // >= 0: static segment [row_begin, row_end); < 0: offsets[dyn], offsets[dyn+1]
  int row_end;
  int dyn;
  const uint16_t* bias; // BF16_PLAIN_BIAS: bf16 [n_out] added before the output is rounded, NULL = none
  int act;              // BF16_PLAIN_BIAS: 0 = none, 1 = erf GELU on the rounded output
  int n_out;            // output features (H for swiglu, N for plain)
  int kbytes;           // bytes per row of a and of the weights
  float* pout;          // split K: row 0 of this group in part 0 of the fp32 partial sums, [parts][rows][n_out]
};

struct GemmArgs {
  GemmGroup g[MAX_GROUPS];
  const int32_t* offsets;  // segment bounds of the dynamic groups, n_offsets + 1 entries
  int n_offsets;
  int G;
  int spread;  // 0: one tile list cut in eighths; 1 / -1: every group cut in eighths, groups walked up / down
  // Split K (plain modes, few tiles): nparts > 1, and every tile of a group exists `parts` times (the entry of `plan`
  // that hdmoe_plan_pick returns for the segment sizes at hand; experts' and static groups are cut differently), part p
  // multiplying K steps [KT*p/parts, KT*(p+1)/parts) and leaving its raw fp32 sums in pout + p * part_stride; a second kernel adds the
  // parts up. 1 = off.
  int nparts;
  long long part_stride;  // floats between two parts
  HdmoeSplitPlan plan;    // split K only
  // Gathered groups only: where *alt.flag reads 0 on the device, their token operand is alt.a (alt.rows rows, row
  // gather[r] >> alt.shift) instead of what the groups say (the gate kernel of the layer picks the layout of the fp8
  // tokens from the scale values and leaves the flag). flag NULL = off.
  HdmoeAltOperand alt;
};

__device__ __forceinline__ int swz(int row) { return ((row >> 1) & 7) ^ ((row & 1) << 2); }

__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, bytes, 0x00020000);
}

typedef __attribute__((address_space(3))) void* lds_ptr_t;

typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

// ---- fp8 K loop in assembly ---------------------------------------------------------------------
// The fragment registers of the fp8 K loop are fixed and its slices are written in assembly: the schedule below
// depends on every fragment being refilled in place right after its last use and on the global->LDS loads of the
// next step being issued one at a time between the MFMAs (the register allocator rotates fragment registers
// and then spills loop-invariant addresses, and a burst of loads behind the barrier keeps both waves of a SIMD
// in the vector-memory issue queue while the matrix pipe runs dry).
//   weight fragments  fb0 v[200:207]  fb1 v[208:215]        token fragments  fa(t) v[216+8t : 223+8t]
// One slice (64 K bytes) = part A (weight half 0 against every token block) + part B (weight half 1). LDS
// requests in flight at the start of a slice, oldest first: fb0, fa0 .. fa(TT-1), fb1 (two ds_read_b128 each);
// LDS returns in order, so part A waits with lgkmcnt(2*(TT-t)) in front of MFMA t. Part B refills fb0 first,
// then fa(t) behind the MFMA that last reads it, then fb1: every fragment is requested TT or more MFMAs (320+
// cycles of matrix pipe) before its first use. The global->LDS loads count on vmcnt, not lgkmcnt.
#define HDMOE_FB0 "v[200:207]"
#define HDMOE_FB1 "v[208:215]"
#define HDMOE_FA0 "v[216:223]"
#define HDMOE_FA1 "v[224:231]"
#define HDMOE_FA2 "v[232:239]"
#define HDMOE_FA3 "v[240:247]"
#define HDMOE_FA4 "v[248:255]"
#define HDMOE_MF(C, A, B) "v_mfma_f32_32x32x64_f8f6f4 %[" C "], " A ", " B ", %[" C "]\n"
// fragment reads: operands w0/w1 (weights) and t0/t1 (tokens) are the lane's two 16-byte halves of the slice read,
// ob / oa the byte offset of the stage read from
#define HDMOE_RD(LO, HI, A0, A1, OFF) \
  "ds_read_b128 " LO ", %[" A0 "] offset:" OFF "\nds_read_b128 " HI ", %[" A1 "] offset:" OFF "\n"
#define HDMOE_RD_FB0 HDMOE_RD("v[200:203]", "v[204:207]", "w0", "w1", "%[ob]")
#define HDMOE_RD_FB1 HDMOE_RD("v[208:211]", "v[212:215]", "w0", "w1", "%[ob]+16384")
#define HDMOE_RD_FA0 HDMOE_RD("v[216:219]", "v[220:223]", "t0", "t1", "%[oa]")
#define HDMOE_RD_FA1 HDMOE_RD("v[224:227]", "v[228:231]", "t0", "t1", "%[oa]+4096")
#define HDMOE_RD_FA2 HDMOE_RD("v[232:235]", "v[236:239]", "t0", "t1", "%[oa]+8192")
#define HDMOE_RD_FA3 HDMOE_RD("v[240:243]", "v[244:247]", "t0", "t1", "%[oa]+12288")
#define HDMOE_RD_FA4 HDMOE_RD("v[248:251]", "v[252:255]", "t0", "t1", "%[oa]+16384")
// one global->LDS load of 8 rows x 128 bytes per wave: M0 = LDS address of the wave's rows (ldsd: the wave's
// offset inside a 64-row slab, IMM: stage and slab), vector offset = the lane's row and chunk, scalar offset = K
#define HDMOE_LD(RS, VO, IMM) \
  "s_add_u32 m0, %[ldsd], " IMM "\ns_nop 0\nbuffer_load_dwordx4 %[" VO "], %[" RS "], %[so] offen lds\n"
#define HDMOE_LDW0 HDMOE_LD("rb0", "vb0", "%[wd]")
#define HDMOE_LDW1 HDMOE_LD("rb0", "vb1", "%[wd]+8192")
#define HDMOE_LDW2 HDMOE_LD("rb1", "vb0", "%[wd]+16384")
#define HDMOE_LDW3 HDMOE_LD("rb1", "vb1", "%[wd]+24576")
#define HDMOE_LDT0 HDMOE_LD("ra", "va0", "%[td]")
#define HDMOE_LDT1 HDMOE_LD("ra", "va1", "%[td]+8192")
#define HDMOE_LDT2 HDMOE_LD("ra", "va2", "%[td]+16384")
#define HDMOE_LDT3 HDMOE_LD("ra", "va3", "%[td]+24576")
#define HDMOE_LDT4 HDMOE_LD("ra", "va4", "%[td]+32768")
#define HDMOE_NONE ""
// part A; L0..L4: what follows each MFMA (a token load of the next step, or nothing)
#define HDMOE_PART_A4(L0, L1, L2, L3)                                                      \
  "s_waitcnt lgkmcnt(8)\n" HDMOE_MF("c0", HDMOE_FB0, HDMOE_FA0) L0                         \
  "s_waitcnt lgkmcnt(6)\n" HDMOE_MF("c1", HDMOE_FB0, HDMOE_FA1) L1                         \
  "s_waitcnt lgkmcnt(4)\n" HDMOE_MF("c2", HDMOE_FB0, HDMOE_FA2) L2                         \
  "s_waitcnt lgkmcnt(2)\n" HDMOE_MF("c3", HDMOE_FB0, HDMOE_FA3) L3
#define HDMOE_PART_A5(L0, L1, L2, L3, L4)                                                  \
  "s_waitcnt lgkmcnt(10)\n" HDMOE_MF("c0", HDMOE_FB0, HDMOE_FA0) L0                        \
  "s_waitcnt lgkmcnt(8)\n" HDMOE_MF("c1", HDMOE_FB0, HDMOE_FA1) L1                         \
  "s_waitcnt lgkmcnt(6)\n" HDMOE_MF("c2", HDMOE_FB0, HDMOE_FA2) L2                         \
  "s_waitcnt lgkmcnt(4)\n" HDMOE_MF("c3", HDMOE_FB0, HDMOE_FA3) L3                         \
  "s_waitcnt lgkmcnt(2)\n" HDMOE_MF("c4", HDMOE_FB0, HDMOE_FA4) L4
#define HDMOE_PART_A4_PLAIN HDMOE_PART_A4(HDMOE_NONE, HDMOE_NONE, HDMOE_NONE, HDMOE_NONE)
#define HDMOE_PART_A5_PLAIN HDMOE_PART_A5(HDMOE_NONE, HDMOE_NONE, HDMOE_NONE, HDMOE_NONE, HDMOE_NONE)
#define HDMOE_PART_A4_LOADS HDMOE_PART_A4(HDMOE_LDT0, HDMOE_LDT1, HDMOE_LDT2, HDMOE_LDT3)
#define HDMOE_PART_A5_LOADS HDMOE_PART_A5(HDMOE_LDT0, HDMOE_LDT1, HDMOE_LDT2, HDMOE_LDT3, HDMOE_LDT4)
// part B with the refills for the next slice; L0..L3: a weight load of the step after the next, or nothing
#define HDMOE_PART_B4(L0, L1, L2, L3)                                                            \
  HDMOE_RD_FB0 "s_waitcnt lgkmcnt(2)\n" HDMOE_MF("d0", HDMOE_FB1, HDMOE_FA0) HDMOE_RD_FA0 L0     \
  HDMOE_MF("d1", HDMOE_FB1, HDMOE_FA1) HDMOE_RD_FA1 L1                                           \
  HDMOE_MF("d2", HDMOE_FB1, HDMOE_FA2) HDMOE_RD_FA2 L2                                           \
  HDMOE_MF("d3", HDMOE_FB1, HDMOE_FA3) HDMOE_RD_FA3 HDMOE_RD_FB1 L3
#define HDMOE_PART_B5(L0, L1, L2, L3)                                                            \
  HDMOE_RD_FB0 "s_waitcnt lgkmcnt(2)\n" HDMOE_MF("d0", HDMOE_FB1, HDMOE_FA0) HDMOE_RD_FA0 L0     \
  HDMOE_MF("d1", HDMOE_FB1, HDMOE_FA1) HDMOE_RD_FA1 L1                                           \
  HDMOE_MF("d2", HDMOE_FB1, HDMOE_FA2) HDMOE_RD_FA2 L2                                           \
  HDMOE_MF("d3", HDMOE_FB1, HDMOE_FA3) HDMOE_RD_FA3 L3                                           \
  HDMOE_MF("d4", HDMOE_FB1, HDMOE_FA4) HDMOE_RD_FA4 HDMOE_RD_FB1
#define HDMOE_PART_B4_PLAIN HDMOE_PART_B4(HDMOE_NONE, HDMOE_NONE, HDMOE_NONE, HDMOE_NONE)
#define HDMOE_PART_B5_PLAIN HDMOE_PART_B5(HDMOE_NONE, HDMOE_NONE, HDMOE_NONE, HDMOE_NONE)
#define HDMOE_PART_B4_LOADS HDMOE_PART_B4(HDMOE_LDW0, HDMOE_LDW1, HDMOE_LDW2, HDMOE_LDW3)
#define HDMOE_PART_B5_LOADS HDMOE_PART_B5(HDMOE_LDW0, HDMOE_LDW1, HDMOE_LDW2, HDMOE_LDW3)
// part B of the last slice of a tile: no refills; the trailing wait states cover the distance the hardware wants
// between the last MFMA and the first VALU read of an accumulator (the compiler cannot see into the block)
#define HDMOE_PART_B4_LAST                                                                                  \
  "s_waitcnt lgkmcnt(0)\n" HDMOE_MF("d0", HDMOE_FB1, HDMOE_FA0) HDMOE_MF("d1", HDMOE_FB1, HDMOE_FA1)        \
  HDMOE_MF("d2", HDMOE_FB1, HDMOE_FA2) HDMOE_MF("d3", HDMOE_FB1, HDMOE_FA3) "s_nop 15\ns_nop 7\n"
#define HDMOE_PART_B5_LAST                                                                                  \
  "s_waitcnt lgkmcnt(0)\n" HDMOE_MF("d0", HDMOE_FB1, HDMOE_FA0) HDMOE_MF("d1", HDMOE_FB1, HDMOE_FA1)        \
  HDMOE_MF("d2", HDMOE_FB1, HDMOE_FA2) HDMOE_MF("d3", HDMOE_FB1, HDMOE_FA3)                                 \
  HDMOE_MF("d4", HDMOE_FB1, HDMOE_FA4) "s_nop 15\ns_nop 7\n"
// Two forms of a part in one block, chosen by the wave-uniform operand fl, so that the accumulators pass through the
// same statement either way (a branch around separate statements makes the compiler copy and spill them).
#define HDMOE_SELECT(IF_SET, IF_CLEAR) \
  "s_cmp_lg_u32 %[fl], 0\ns_cbranch_scc0 1f\n" IF_SET "s_branch 2f\n1:\n" IF_CLEAR "2:\n"
// the first fragments of a tile, in the order the waits of part A assume
#define HDMOE_FILL4 HDMOE_RD_FB0 HDMOE_RD_FA0 HDMOE_RD_FA1 HDMOE_RD_FA2 HDMOE_RD_FA3 HDMOE_RD_FB1
#define HDMOE_FILL5 HDMOE_RD_FB0 HDMOE_RD_FA0 HDMOE_RD_FA1 HDMOE_RD_FA2 HDMOE_RD_FA3 HDMOE_RD_FA4 HDMOE_RD_FB1

// LIGHT (fp8 only): the K loop is the compiler-scheduled one of the 16-bit modes, which skips the 32-token blocks of a
// tile that hold no rows, instead of the assembly loop, which multiplies padding like rows. For launches whose tiles are
// mostly padding (few tokens per segment).
template <int MODE, int TT, bool LIGHT = false>
__global__ __launch_bounds__(NTHREADS) void grouped_gemm_kernel(const GemmArgs args) {
  constexpr bool FP8 = (MODE == FP8_SWIGLU || MODE == FP8_PLAIN || MODE == FP8_PLAIN_BIAS);
  constexpr bool SWIGLU = (MODE == FP8_SWIGLU || MODE == BF16_SWIGLU);
  constexpr bool BIAS = (MODE == BF16_PLAIN_BIAS || MODE == FP8_PLAIN_BIAS || MODE == F16_PLAIN_BIAS);  // Linear with bias and optional GELU
  constexpr bool F16 = MODE == F16_PLAIN_BIAS;
  using Act = std::conditional_t<F16, HdmoeF16, HdmoeBf16>;  // element format of activations, bias and outputs
  constexpr int WAVE_TOK = 32 * TT;        // tokens per wave row
  constexpr int BM = 2 * WAVE_TOK;         // tokens per block tile
  constexpr int A_SLABS = BM / 64;         // 64-row slabs of the token tile
  constexpr int A_BYTES = BM * BK;         // token tile of one K step in LDS; the weight tile follows it
  constexpr int STAGE_BYTES = (BM + BN) * BK;
  constexpr int FEAT_PER_TILE = SWIGLU ? BN / 2 : BN;  // output features per block tile
  // LDS layout of the two stages. bf16: stage after stage, [A0 | B0 | A1 | B1]. fp8: [A0 | A1 | B0 | B1], so that
  // every fragment read of the K loop is one of eight per-lane base addresses plus an immediate below 64 KiB.
  constexpr int B_BYTES = BN * BK;
  constexpr int A_OFF1 = FP8 ? A_BYTES : STAGE_BYTES;
  constexpr int B_OFF0 = FP8 ? 2 * A_BYTES : A_BYTES;
  constexpr int B_OFF1 = FP8 ? 2 * A_BYTES + B_BYTES : STAGE_BYTES + A_BYTES;
  // RING3 (the light form on the 128-token tile; split K only): three stages [A | B] one after the other, K steps
  // requested two ahead. With few rows a K step lasts as long as its loads take to arrive, not as long as its MFMAs.
  constexpr bool RING3 = LIGHT && TT == 2;
  static_assert(!RING3 || !BIAS, "the three-stage ring is built for the feed-forward contractions");
  static_assert(TT != 2 || RING3, "the 128-token tile exists only with the three-stage ring");
  auto a_off = [](int stage) { return RING3 ? stage * STAGE_BYTES : (stage ? A_OFF1 : 0); };
  auto b_off = [](int stage) { return RING3 ? stage * STAGE_BYTES + A_BYTES : (stage ? B_OFF1 : B_OFF0); };
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  if constexpr (RING3 && !SWIGLU) {
    if (args.nparts <= 1) return;  // its plain epilogue is the partial-sum store only (kernel argument: uniform)
  }

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // wave-uniform by construction
  const int wq = wave & 3, wt = wave >> 2;

  // ---- tile enumeration (persistent blocks) ----------------------------------------------
  // Segment bounds of the dynamic groups: one vector load, then lane reads.
  int off_lane = 0;
  if (args.offsets != nullptr && lane <= args.n_offsets) off_lane = args.offsets[lane];
  auto seg = [&](const GemmGroup& gg, int& rb, int& re) {
    if (gg.row_begin >= 0) { rb = gg.row_begin; re = gg.row_end; }
    else { rb = __builtin_amdgcn_readlane(off_lane, gg.dyn); re = __builtin_amdgcn_readlane(off_lane, gg.dyn + 1); }
  };
  // the gathered token operand: as the groups describe it, or the alternative the flag selects
  const bool use_alt = args.alt.flag != nullptr && __builtin_amdgcn_readfirstlane(*args.alt.flag) == 0;
  auto gathered_a = [&](const GemmGroup& gg) { return use_alt ? args.alt.a : gg.a; };
  auto gathered_rows = [&](const GemmGroup& gg) { return use_alt ? args.alt.rows : gg.a_rows; };
  auto gathered_shift = [&](const GemmGroup& gg) { return use_alt ? args.alt.shift : gg.gather_shift; };
  // split K: which cut of the plan runs (a function of the segment sizes; the kernel that adds the parts up makes the
  // same choice)
  int plan_idx = 0;
  if (args.nparts > 1 && args.plan.n > 1) {
    int mt_dyn = 0, mt_static = 0;
    for (int g = 0; g < args.G; ++g) {
      int rb, re;
      seg(args.g[g], rb, re);
      const int mt = (re - rb + args.plan.bm - 1) / args.plan.bm;  // the plan's own tile height: the other kernel's count
      if (args.g[g].row_begin < 0) mt_dyn += mt;
      else mt_static += mt;
    }
    plan_idx = hdmoe_plan_pick(args.plan, mt_dyn, mt_static, args.g[0].n_out / FEAT_PER_TILE);
  }
  const int parts_dyn = args.nparts > 1 ? args.plan.pd[plan_idx] : 1, parts_static = args.nparts > 1 ? args.plan.ps[plan_idx] : 1;
  auto parts_of = [&](int g) { return args.g[g].row_begin < 0 ? parts_dyn : parts_static; };
  int total = 0;
  for (int g = 0; g < args.G; ++g) {
    int rb, re;
    seg(args.g[g], rb, re);
    total += ((re - rb + BM - 1) / BM) * (args.g[g].n_out / FEAT_PER_TILE) * parts_of(g);
  }
  // Each XCD (block ids congruent mod 8) walks one contiguous eighth of the tile list and its blocks take
  // consecutive tiles, so the CUs of an XCD share operand tiles in their L2.
  const int per_xcd = (total + HDMOE_NUM_XCD - 1) / HDMOE_NUM_XCD;
  const int xcd = blockIdx.x % HDMOE_NUM_XCD, slot = blockIdx.x / HDMOE_NUM_XCD;
  const int nslots = gridDim.x / HDMOE_NUM_XCD;

  struct Tile { int g, row0, rows_here, n0, kbytes, part, kt0, nkt; };
  auto decode = [&](int i) -> Tile {
    Tile d = {-1, 0, 0, 0, 0, 0, 0, 0};
    int in_xcd = slot + i * nslots;
    int L = 0, g = 0, rb = 0, re = 0, mtiles = 0, ntiles = 0;
    if (args.spread != 0) {
      // Groups whose tiles differ in length (the K of the shared expert's down projection is about half the
      // routed experts'): every XCD takes its eighth of every group, longest tiles first, so each block gets
      // the same mix and the blocks end together.
      int k = 0;
      for (; k < args.G; ++k) {
        g = args.spread > 0 ? k : args.G - 1 - k;
        seg(args.g[g], rb, re);
        mtiles = (re - rb + BM - 1) / BM;
        ntiles = args.g[g].n_out / FEAT_PER_TILE;
        const long long tiles = (long long)mtiles * ntiles * parts_of(g);
        const int lo = (int)(xcd * tiles / HDMOE_NUM_XCD), hi = (int)((xcd + 1) * tiles / HDMOE_NUM_XCD);
        if (in_xcd < hi - lo) { L = lo + in_xcd; break; }
        in_xcd -= hi - lo;
      }
      if (k >= args.G) return d;
    } else {
      L = xcd * per_xcd + in_xcd;
      if (in_xcd >= per_xcd || L >= total) return d;
      for (; g < args.G; ++g) {
        seg(args.g[g], rb, re);
        mtiles = (re - rb + BM - 1) / BM;
        ntiles = args.g[g].n_out / FEAT_PER_TILE;
        const int tiles = mtiles * ntiles * parts_of(g);
        if (L < tiles) break;
        L -= tiles;
      }
      if (g >= args.G) return d;
    }
    // split K: the parts of a group one after the other (tiles of one part share operand slices, parts do not)
    const int part = L / (mtiles * ntiles);
    L -= part * (mtiles * ntiles);
    // bands of GROUP_M m-tiles; a short remainder joins the last band, so that the cheap partial m-tile at the
    // end of a segment is interleaved with full ones instead of forming a run of its own
    const int nbands = max(1, (mtiles + GROUP_M / 2) / GROUP_M);
    const int band = min(L / (GROUP_M * ntiles), nbands - 1);
    const int first_m = band * GROUP_M;
    const int gm = band == nbands - 1 ? mtiles - first_m : GROUP_M;
    const int within = L - band * (GROUP_M * ntiles);
    d.g = g;
    d.row0 = rb + (first_m + within % gm) * BM;
    d.rows_here = min(re - d.row0, BM);
    d.n0 = (within / gm) * FEAT_PER_TILE;
    d.kbytes = args.g[g].kbytes;
    const int ktf = d.kbytes / BK;
    d.part = part;
    d.kt0 = ktf * part / parts_of(g);
    d.nkt = ktf * (part + 1) / parts_of(g) - d.kt0;
    return d;
  };

  // ---- global -> LDS addressing --------------------------------------------------
  // One wave-level load moves 8 rows x 128 bytes. Lane i lands in LDS chunk (i&7) of row (i>>3) and therefore
  // fetches logical chunk (i&7) ^ f(row). Rows past the segment end are outside the buffer range and read as
  // zero: the row part of the address sits in the VGPR offset, the only one that is range-checked; the K
  // position goes through the scalar offset.
  const int ld_row = wave * 8 + (lane >> 3);                 // row within a 64-row slab
  const int ld_chunk = (lane & 7) ^ swz(ld_row);
  const int ld_lds = wave * 8 * BK;                          // + slab*64*BK

  // source of the tile being loaded (buffer resources are kept as plain locals: the opaque resource type
  // cannot be a struct member)
  //
  // Weight rows of the tile. SwiGLU: LDS half h (128 rows) holds rows n0..n0+127 of w1 (h=0) / w3 (h=1).
  // Plain: wave column wq multiplies LDS rows wq*32..+32 of both halves, and its 64 output features should be
  // contiguous in memory, so LDS row (h, wq, i) holds weight row n0 + wq*64 + h*32 + i.
  __amdgpu_buffer_rsrc_t src_a = make_rsrc(nullptr, 0), src_b0 = src_a, src_b1 = src_a;
  int src_voff[MAX_SLABS] = {};
  int src_voff_b[2] = {0, 0};
  // Row indices of a gathered token operand: loaded one tile ahead (load_gather), consumed by set_src.
  auto load_gather = [&](const Tile& d, int (&gi)[MAX_SLABS]) {
    const GemmGroup& gg = args.g[d.g];
#pragma unroll
    for (int j = 0; j < A_SLABS; ++j) {
      const int r = j * 64 + ld_row;
      gi[j] = (gg.gather != nullptr && r < d.rows_here) ? (gg.gather[d.row0 + r] >> gathered_shift(gg)) : -1;
    }
  };
  // the same three resources as plain descriptor words, for the loads issued from the assembly blocks
  [[maybe_unused]] v4i ra4 = {0, 0, 0, 0}, rb04 = ra4, rb14 = ra4;
  auto raw_rsrc = [](const void* p, uint32_t bytes) -> v4i {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    v4i r;
    r.x = (int)(uint32_t)a; r.y = (int)(uint32_t)((a >> 32) & 0xffffu); r.z = (int)bytes; r.w = 0x00020000;
    return r;
  };
  int k_base = 0;  // K byte offset of step 0 of the tile being loaded (split K)
  auto set_src = [&](const Tile& d, const int (&gi)[MAX_SLABS]) {
    const GemmGroup& gg = args.g[d.g];
    k_base = d.kt0 * BK;
    if constexpr (FP8) {
      if (gg.gather != nullptr) ra4 = raw_rsrc(gathered_a(gg), (uint32_t)gathered_rows(gg) * (uint32_t)d.kbytes);
      else ra4 = raw_rsrc(gg.a + (size_t)d.row0 * d.kbytes, (uint32_t)d.rows_here * (uint32_t)d.kbytes);
      const uint32_t wrows = SWIGLU ? BN / 2 : BN - 32;
      rb04 = raw_rsrc(gg.b0 + (size_t)d.n0 * d.kbytes, wrows * (uint32_t)d.kbytes);
      rb14 = raw_rsrc(SWIGLU ? gg.b1 + (size_t)d.n0 * d.kbytes : gg.b0 + (size_t)(d.n0 + 32) * d.kbytes,
                      wrows * (uint32_t)d.kbytes);
    }
    if (gg.gather != nullptr) {
      // rows past the segment end get an offset beyond the buffer and read as zero
      src_a = make_rsrc(gathered_a(gg), (uint32_t)gathered_rows(gg) * (uint32_t)d.kbytes);
#pragma unroll
      for (int j = 0; j < A_SLABS; ++j) src_voff[j] = gi[j] >= 0 ? gi[j] * d.kbytes + ld_chunk * 16 : (int)0x80000000u;
    } else {
      src_a = make_rsrc(gg.a + (size_t)d.row0 * d.kbytes, (uint32_t)d.rows_here * (uint32_t)d.kbytes);
#pragma unroll
      for (int j = 0; j < A_SLABS; ++j) src_voff[j] = (j * 64 + ld_row) * d.kbytes + ld_chunk * 16;
    }
    const uint8_t* b_half0 = gg.b0 + (size_t)d.n0 * d.kbytes;
    const uint8_t* b_half1 = SWIGLU ? gg.b1 + (size_t)d.n0 * d.kbytes : gg.b0 + (size_t)(d.n0 + 32) * d.kbytes;
    const uint32_t b_rows = SWIGLU ? BN / 2 : BN - 32;
    src_b0 = make_rsrc(b_half0, b_rows * (uint32_t)d.kbytes);
    src_b1 = make_rsrc(b_half1, b_rows * (uint32_t)d.kbytes);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int r = j * 64 + ld_row;  // row within the 128-row LDS half
      src_voff_b[j] = (SWIGLU ? r : (r >> 5) * 64 + (r & 31)) * d.kbytes + ld_chunk * 16;
    }
  };
  // K steps of the tile being loaded; a step at or past it (padding) is fetched as zeros. Step 0 of a tile is
  // requested before the tile becomes current, so the count is never below 1.
  int kt_real = 1;
  auto issue_loads = [&](int stage, int kt) {
    uint8_t* sa = smem + a_off(stage);
    uint8_t* sb = smem + b_off(stage);
    const int k0 = k_base + kt * BK;
    const __amdgpu_buffer_rsrc_t empty = make_rsrc(nullptr, 0);
    const bool pad = kt >= kt_real;
    const __amdgpu_buffer_rsrc_t ra = pad ? empty : src_a, rb0 = pad ? empty : src_b0, rb1 = pad ? empty : src_b1;
#pragma unroll
    for (int j = 0; j < A_SLABS; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(ra, (lds_ptr_t)(sa + ld_lds + j * 64 * BK), 16, src_voff[j], k0, 0, 0);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb0, (lds_ptr_t)(sb + ld_lds + j * 64 * BK), 16, src_voff_b[j], k0, 0, 0);
#pragma unroll
    for (int j = 0; j < 2; ++j)
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rb1, (lds_ptr_t)(sb + ld_lds + (j + 2) * 64 * BK), 16, src_voff_b[j], k0, 0, 0);
  };

  // ---- LDS -> MFMA fragment addressing -------------------------------------------
  // Operand tile of 32 rows: lane l reads row (l&31); its K sub-block is (l>>5).
  const int fr_row = lane & 31;
  const int fr_grp = lane >> 5;
  const int fr_swz = swz(fr_row);  // tile origins are multiples of 32 rows, so f() only sees fr_row
  const int a_base = (wt * WAVE_TOK + fr_row) * BK;          // token operand within its stage, + tt*32*BK
  const int b_base = (wq * 32 + fr_row) * BK;                // weight operand within its stage, + ft*128*BK

  v16f acc[2][TT];
  // n_tt: how many of this wave's four 32-token blocks hold rows of the tile (4 except in the last, partial
  // m-tile of a segment); the others are neither read from LDS nor multiplied.
  [[maybe_unused]] auto compute = [&](int stage, auto full_c, int n_tt) {
    constexpr bool FULL = decltype(full_c)::value;
    const uint8_t* sa = smem + a_off(stage) + a_base;
    const uint8_t* sb = smem + b_off(stage) + b_base;
    if constexpr (!FP8) {
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const int c0 = ((ks * 2 + fr_grp) ^ fr_swz) * 16;
        using frag_t = std::conditional_t<F16, v8h, v8bf>;
        frag_t fa[TT], fb[2];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          if (!FULL && tt >= n_tt) continue;
          fa[tt] = *reinterpret_cast<const frag_t*>(sa + tt * 32 * BK + c0);
        }
        if (!FULL && n_tt == 0) continue;
#pragma unroll
        for (int ft = 0; ft < 2; ++ft)
          fb[ft] = *reinterpret_cast<const frag_t*>(sb + ft * 128 * BK + c0);
#pragma unroll
        for (int ft = 0; ft < 2; ++ft)
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            if (!FULL && tt >= n_tt) continue;
            if constexpr (F16) acc[ft][tt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fb[ft], fa[tt], acc[ft][tt], 0, 0, 0);
            else acc[ft][tt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fb[ft], fa[tt], acc[ft][tt], 0, 0, 0);
          }
      }
    } else {
      // fp8: the fragments, MFMA and order over K of the assembly loop below (slice 0 then slice 1 of a step into the
      // same accumulator), scheduled by the compiler
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const int c0 = ((ks * 4 + fr_grp * 2) ^ fr_swz) * 16;
        auto frag = [&](const uint8_t* p) {
          const v4i lo = *reinterpret_cast<const v4i*>(p + c0), hi = *reinterpret_cast<const v4i*>(p + (c0 ^ 16));
          const v8i f = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
          return f;
        };
        v8i fa[TT], fb[2];
#pragma unroll
        for (int tt = 0; tt < TT; ++tt) {
          if (!FULL && tt >= n_tt) continue;
          fa[tt] = frag(sa + tt * 32 * BK);
        }
        if (!FULL && n_tt == 0) continue;
#pragma unroll
        for (int ft = 0; ft < 2; ++ft) fb[ft] = frag(sb + ft * 128 * BK);
#pragma unroll
        for (int ft = 0; ft < 2; ++ft)
#pragma unroll
          for (int tt = 0; tt < TT; ++tt) {
            if (!FULL && tt >= n_tt) continue;
            acc[ft][tt] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb[ft], fa[tt], acc[ft][tt], 0, 0, 0, 0, 0, 0);
          }
      }
    }
  };

  // ---- fp8: software-pipelined K loop in assembly (macros above the kernel) --------------------------------
  [[maybe_unused]] v8i fb0, fb1, fa0, fa1, fa2, fa3, fa4;
  [[maybe_unused]] uint32_t tok_addr[2][2], w_addr[2][2];  // LDS byte address of this lane's reads, [slice][16-byte half]
  if constexpr (FP8) {
    const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int c = (((ks * 4 + fr_grp * 2) ^ fr_swz) * 16) ^ (h * 16);
        tok_addr[ks][h] = lds0 + a_base + c;
        w_addr[ks][h] = lds0 + B_OFF0 + b_base + c;
      }
  }
#define HDMOE_FRAGS4                                                                                           \
  "+{v[200:207]}"(fb0), "+{v[208:215]}"(fb1), "+{v[216:223]}"(fa0), "+{v[224:231]}"(fa1), "+{v[232:239]}"(fa2), \
      "+{v[240:247]}"(fa3)
#define HDMOE_FRAGS5 HDMOE_FRAGS4, "+{v[248:255]}"(fa4)
#define HDMOE_FRAGS4_OUT                                                                                       \
  "={v[200:207]}"(fb0), "={v[208:215]}"(fb1), "={v[216:223]}"(fa0), "={v[224:231]}"(fa1), "={v[232:239]}"(fa2), \
      "={v[240:247]}"(fa3)
#define HDMOE_FRAGS5_OUT HDMOE_FRAGS4_OUT, "={v[248:255]}"(fa4)
#define HDMOE_ACC_A4 [c0] "+v"(acc[0][0]), [c1] "+v"(acc[0][1]), [c2] "+v"(acc[0][2]), [c3] "+v"(acc[0][3])
#define HDMOE_ACC_B4 [d0] "+v"(acc[1][0]), [d1] "+v"(acc[1][1]), [d2] "+v"(acc[1][2]), [d3] "+v"(acc[1][3])
#define HDMOE_ACC_A5 HDMOE_ACC_A4, [c4] "+v"(acc[0][TT - 1])
#define HDMOE_ACC_B5 HDMOE_ACC_B4, [d4] "+v"(acc[1][TT - 1])
  // fragment reads of slice KS out of stage SS
#define HDMOE_SRC(KS, SS)                                                                                      \
  [w0] "v"(w_addr[KS][0]), [w1] "v"(w_addr[KS][1]), [t0] "v"(tok_addr[KS][0]), [t1] "v"(tok_addr[KS][1]),      \
      [oa] "i"((SS) * A_BYTES), [ob] "i"((SS) * B_BYTES)
  // token loads into stage TS: resource, the lane offsets of the slabs, K offset, the wave's LDS offset
#define HDMOE_TOK_LOADS(TS)                                                                                    \
  [fl] "s"(fl), [ra] "s"(ra), [so] "s"(so), [ldsd] "s"(lds_wave), [td] "i"((TS) ? A_OFF1 : 0),                 \
      [va0] "v"(src_voff[0]), [va1] "v"(src_voff[1]), [va2] "v"(src_voff[2]), [va3] "v"(src_voff[3]),          \
      [va4] "v"(src_voff[A_SLABS - 1])
  // weight loads into stage WS
#define HDMOE_W_LOADS(WS)                                                                                      \
  [fl] "s"(fl), [rb0] "s"(rb0), [rb1] "s"(rb1), [so] "s"(so), [ldsd] "s"(lds_wave),                            \
      [wd] "i"((WS) ? B_OFF1 : B_OFF0), [vb0] "v"(src_voff_b[0]), [vb1] "v"(src_voff_b[1])
  [[maybe_unused]] uint32_t lds_wave = 0;  // LDS address of this wave's rows inside a 64-row slab of stage 0's token tile
  if constexpr (FP8) lds_wave = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(lds_ptr_t)smem + ld_lds);
  // the tile's first fragments: slice 0 of stage 0
  [[maybe_unused]] auto fp8_fill = [&] {
    if constexpr (FP8 && TT == 5) asm volatile(HDMOE_FILL5 : HDMOE_FRAGS5_OUT : HDMOE_SRC(0, 0) : "memory");
    else if constexpr (FP8) asm volatile(HDMOE_FILL4 : HDMOE_FRAGS4_OUT : HDMOE_SRC(0, 0) : "memory");
  };
  [[maybe_unused]] auto fp8_a = [&] {
    if constexpr (FP8 && TT == 5) asm volatile(HDMOE_PART_A5_PLAIN : HDMOE_ACC_A5, HDMOE_FRAGS5 : : "memory");
    else if constexpr (FP8) asm volatile(HDMOE_PART_A4_PLAIN : HDMOE_ACC_A4, HDMOE_FRAGS4 : : "memory");
  };
  // part A that, if fl is set, also requests the token rows of K offset so into stage TS, one load behind each MFMA
#define HDMOE_DEF_PART_A_LOADS(NAME, TS)                                                                        \
  [[maybe_unused]] auto NAME = [&](int fl, v4i ra, int so) {                                                    \
    if constexpr (FP8 && TT == 5)                                                                               \
      asm volatile(HDMOE_SELECT(HDMOE_PART_A5_LOADS, HDMOE_PART_A5_PLAIN)                                       \
                   : HDMOE_ACC_A5, HDMOE_FRAGS5 : HDMOE_TOK_LOADS(TS) : "memory", "scc");                       \
    else if constexpr (FP8)                                                                                     \
      asm volatile(HDMOE_SELECT(HDMOE_PART_A4_LOADS, HDMOE_PART_A4_PLAIN)                                       \
                   : HDMOE_ACC_A4, HDMOE_FRAGS4 : HDMOE_TOK_LOADS(TS) : "memory", "scc");                       \
  }
  HDMOE_DEF_PART_A_LOADS(fp8_a_loads_to0, 0);
  HDMOE_DEF_PART_A_LOADS(fp8_a_loads_to1, 1);
  // part B with the refills from slice KS of stage SS
#define HDMOE_DEF_PART_B(NAME, SS, KS)                                                                          \
  [[maybe_unused]] auto NAME = [&] {                                                                            \
    if constexpr (FP8 && TT == 5)                                                                               \
      asm volatile(HDMOE_PART_B5_PLAIN : HDMOE_ACC_B5, HDMOE_FRAGS5 : HDMOE_SRC(KS, SS) : "memory");            \
    else if constexpr (FP8)                                                                                     \
      asm volatile(HDMOE_PART_B4_PLAIN : HDMOE_ACC_B4, HDMOE_FRAGS4 : HDMOE_SRC(KS, SS) : "memory");            \
  }
  HDMOE_DEF_PART_B(fp8_b_s0k1, 0, 1);
  HDMOE_DEF_PART_B(fp8_b_s1k1, 1, 1);
  // second slice of an even step: refills from slice 0 of stage 1; if fl is set, the weight rows of K offset so
  // go into stage 0
  [[maybe_unused]] auto fp8_b_even = [&](int fl, v4i rb0, v4i rb1, int so) {
    if constexpr (FP8 && TT == 5)
      asm volatile(HDMOE_SELECT(HDMOE_PART_B5_LOADS, HDMOE_PART_B5_PLAIN)
                   : HDMOE_ACC_B5, HDMOE_FRAGS5 : HDMOE_SRC(0, 1), HDMOE_W_LOADS(0) : "memory", "scc");
    else if constexpr (FP8)
      asm volatile(HDMOE_SELECT(HDMOE_PART_B4_LOADS, HDMOE_PART_B4_PLAIN)
                   : HDMOE_ACC_B4, HDMOE_FRAGS4 : HDMOE_SRC(0, 1), HDMOE_W_LOADS(0) : "memory", "scc");
  };
  // second slice of an odd step: if fl is set (another pair of steps follows), refills from slice 0 of stage 0 and
  // the weight rows of K offset so go into stage 1; else it is the last slice of the tile
  [[maybe_unused]] auto fp8_b_odd = [&](int fl, v4i rb0, v4i rb1, int so) {
    if constexpr (FP8 && TT == 5)
      asm volatile(HDMOE_SELECT(HDMOE_PART_B5_LOADS, HDMOE_PART_B5_LAST)
                   : HDMOE_ACC_B5, HDMOE_FRAGS5 : HDMOE_SRC(0, 0), HDMOE_W_LOADS(1) : "memory", "scc");
    else if constexpr (FP8)
      asm volatile(HDMOE_SELECT(HDMOE_PART_B4_LOADS, HDMOE_PART_B4_LAST)
                   : HDMOE_ACC_B4, HDMOE_FRAGS4 : HDMOE_SRC(0, 0), HDMOE_W_LOADS(1) : "memory", "scc");
  };

  // ---- epilogue ----------------------------------------------------------------------
  // acc[ft][tt][i]: feature = (i>>2)*8 + (lane>>5)*4 + (i&3) within the 32-row MFMA tile (ft = weight half),
  // token = lane&31 within the 32-token MFMA tile: a lane owns 4 consecutive features of one token, and one store
  // instruction issued from that layout would touch 32 different rows with 8 or 16 bytes each. The packed values
  // therefore go through LDS (stage 1, free once the K loop is over) and leave as 16 bytes per lane, 8 lanes to
  // a 128-byte row piece. Staging rows are 128 bytes (256 for bf16 SwiGLU) with the 16-byte chunk index XORed
  // with (token & 7). Stores go through a buffer resource covering exactly the valid rows of the tile: rows past
  // the segment end are dropped by the range check.
  const int tok32 = lane & 31;
  const int hi32 = lane >> 5;
  // Staging room for the outputs once the K loop is over: whatever is not stage 0 (which takes the next tile's
  // first K step meanwhile). fp8: the token tile of stage 1 (BM x 128 bytes: exactly the SwiGLU tile) and the
  // weight tile of stage 1; bf16: stage 1 as a whole.
  // (three-stage ring: the token tile of stage 2; the next tile's first two K steps go to stages 0 and 1 meanwhile)
  uint8_t* const stg = smem + (RING3 ? 2 * STAGE_BYTES : FP8 ? A_OFF1 : STAGE_BYTES);
  auto wave_sync = [] {
    // orders this wave's LDS writes before its LDS reads of other lanes' data (LDS executes a wave's requests
    // in order; this only stops the compiler from moving them)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  };
  // Per-tile epilogue factors. They are loaded before the K loop: a load issued after the next tile's
  // global->LDS requests would make the epilogue wait for those as well (one in-order counter).
  float ep_a = 1.0f, ep_b = 1.0f, ep_next = 1.0f;
  u32x2 ep_bias[2][4];  // BIAS: the 2 x 4 feature quads of this lane, 4 bf16 each
  auto load_scales = [&](const Tile& d) {
    if constexpr (BIAS) {
      const GemmGroup& gg = args.g[d.g];
#pragma unroll
      for (int ft = 0; ft < 2; ++ft)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          u32x2 z = {0u, 0u};
          if (gg.bias != nullptr)
            z = *reinterpret_cast<const u32x2*>(gg.bias + d.n0 + wq * 64 + ft * 32 + q * 8 + (lane >> 5) * 4);
          ep_bias[ft][q] = z;
        }
    }
    if constexpr (FP8) {
      const GemmGroup& gg = args.g[d.g];
      const float s_in = gg.s_in ? *gg.s_in : 1.0f;
      ep_a = s_in * *gg.sb0;
      if constexpr (SWIGLU) {
        ep_b = (gg.s_in_b ? *gg.s_in_b : s_in) * *gg.sb1;
        ep_next = gg.s_next ? hdmoe_dev_round_bf16(__fdiv_rn(1.0f, *gg.s_next)) : -1.0f;
      }
    }
  };
  auto round2_bf16 = [](float& a, float& b) {
    const uint32_t p = hdmoe_dev_pack_bf16(a, b);
    a = __uint_as_float(p << 16);
    b = __uint_as_float(p & 0xffff0000u);
  };
  auto epilogue = [&](const Tile& d) {
    const GemmGroup& gg = args.g[d.g];
    if constexpr (SWIGLU) {
      const float sg = ep_a, su = ep_b, inv_next = ep_next;
      constexpr int EB = FP8 ? 1 : 2;
      constexpr int ROWB = (BN / 2) * EB;  // bytes of one staged token row: the tile's 128 features
      const int ldo = gg.n_out * EB;
      const __amdgpu_buffer_rsrc_t ro = make_rsrc(gg.out + (size_t)d.row0 * ldo, (uint32_t)d.rows_here * (uint32_t)ldo);
      // The cast in front of the w2 Linear (ops.py:337-343) has three forms, fixed per tile: clamp to +-448 when
      // that Linear has no scale_input, nothing when 1/scale_input is 1, else multiply and round. The choice is
      // made once, outside the element loop.
      // bf16 with the 320-token tile: 320 rows of 256 bytes are more than stage 1 holds, so the tile is staged and
      // stored in two passes, the first three 32-token blocks of either wave row, then the last two.
      constexpr bool TWO_PASS = !FP8 && TT == 5;
      auto swiglu_tile = [&](auto next_mode, auto pass_c) {
        constexpr int NEXT = decltype(next_mode)::value;  // 0 clamp, 1 unit scale, 2 general scale
        constexpr int PASS = decltype(pass_c)::value;     // -1: all blocks in one go; 0, 1: the passes of TWO_PASS
        constexpr int TT0 = PASS == 1 ? 3 : 0, TT1 = PASS == 0 ? 3 : TT;
#pragma unroll
        for (int tt = TT0; tt < TT1; ++tt) {
          const int tok = PASS < 0 ? wt * WAVE_TOK + tt * 32 + tok32 : wt * ((TT1 - TT0) * 32) + (tt - TT0) * 32 + tok32;
          uint8_t* const row = stg + tok * ROWB;
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            float m[4];
            uint32_t pm[2];  // the same four values as packed bf16 pairs (fp8 cast without unpacking them again)
#pragma unroll
            for (int i = 0; i < 4; i += 2) {
              // two elements at a time: one packed conversion rounds both to bf16
              float h1a = acc[0][tt][q * 4 + i] * sg, h1b = acc[0][tt][q * 4 + i + 1] * sg;   // w1(x)
              float h3a = acc[1][tt][q * 4 + i] * su, h3b = acc[1][tt][q * 4 + i + 1] * su;   // w3(x)
              round2_bf16(h1a, h1b);
              round2_bf16(h3a, h3b);
              float sa = h1a * __builtin_amdgcn_rcpf(1.0f + __expf(-h1a));                     // silu(.)
              float sb = h1b * __builtin_amdgcn_rcpf(1.0f + __expf(-h1b));
              round2_bf16(sa, sb);
              float ma = sa * h3a, mb = sb * h3b;                                              // silu(.) * w3(x)
              if constexpr (FP8 && NEXT == 1) {
                pm[i / 2] = hdmoe_dev_pack_bf16(ma, mb);  // the rounding to bf16; cast from the packed pair below
              } else {
                round2_bf16(ma, mb);
              }
              if constexpr (FP8 && NEXT == 2) {
                ma *= inv_next;
                mb *= inv_next;
                pm[i / 2] = hdmoe_dev_pack_bf16(ma, mb);
              }
              if constexpr (FP8 && NEXT == 0) {
                ma = ma < -448.0f ? -448.0f : (ma > 448.0f ? 448.0f : ma);
                mb = mb < -448.0f ? -448.0f : (mb > 448.0f ? 448.0f : mb);
              }
              m[i] = ma;
              m[i + 1] = mb;
            }
            const int byte = (wq * 32 + q * 8 + hi32 * 4) * EB;  // position of the 4 features in the staged row
            uint8_t* const dst = row + ((((byte >> 4) ^ (tok32 & 7)) << 4) | (byte & 15));
            if constexpr (FP8 && NEXT != 0) {
              *reinterpret_cast<uint32_t*>(dst) = hdmoe_dev_pack4_e4m3fn_bf16(pm[0], pm[1]);
            } else if constexpr (FP8) {
              *reinterpret_cast<uint32_t*>(dst) = hdmoe_dev_pack4_e4m3fn(m[0], m[1], m[2], m[3]);
            } else {
              u32x2 pk;
              pk.x = hdmoe_dev_pack_bf16(m[0], m[1]);
              pk.y = hdmoe_dev_pack_bf16(m[2], m[3]);
              *reinterpret_cast<u32x2*>(dst) = pk;
            }
          }
        }
      };
      constexpr int LANES_PER_ROW = ROWB / 16;
      constexpr int ROWS_PER_PASS = 64 / LANES_PER_ROW;
      const int c = lane % LANES_PER_ROW;
      constexpr std::integral_constant<int, -1> all_blocks{};
      if constexpr (TWO_PASS) {
        auto store_pass = [&](auto pass_c) {
          constexpr int PASS = decltype(pass_c)::value;
          constexpr int TT0 = PASS == 1 ? 3 : 0, NTT = PASS == 0 ? 3 : TT - 3;
          swiglu_tile(std::integral_constant<int, 1>{}, pass_c);
          __syncthreads();  // this pass's 2 x NTT x 32 rows are staged
#pragma unroll
          for (int p = 0; p < (NTT * 8) / ROWS_PER_PASS; ++p) {
            const int rl = wave * (NTT * 8) + p * ROWS_PER_PASS + lane / LANES_PER_ROW;    // staged row
            const int r = (rl / (NTT * 32)) * WAVE_TOK + TT0 * 32 + rl % (NTT * 32);        // row of the tile
            const v4i v = *reinterpret_cast<const v4i*>(stg + rl * ROWB + ((c ^ (rl & 7)) << 4));
            __builtin_amdgcn_raw_buffer_store_b128(v, ro, r * ldo + d.n0 * EB + c * 16, 0, 0);
          }
        };
        store_pass(std::integral_constant<int, 0>{});
        __syncthreads();  // everyone has read the first pass's rows
        store_pass(std::integral_constant<int, 1>{});
      } else {
        if constexpr (FP8) {
          const int next = __builtin_amdgcn_readfirstlane(inv_next < 0.0f ? 0 : (inv_next == 1.0f ? 1 : 2));
          if (next == 0) swiglu_tile(std::integral_constant<int, 0>{}, all_blocks);
          else if (next == 1) swiglu_tile(std::integral_constant<int, 1>{}, all_blocks);
          else swiglu_tile(std::integral_constant<int, 2>{}, all_blocks);
        } else {
          swiglu_tile(std::integral_constant<int, 1>{}, all_blocks);
        }
        __syncthreads();  // the tile's 256 x 128 outputs are staged
#pragma unroll
        for (int p = 0; p < (BM / 8) / ROWS_PER_PASS; ++p) {
          const int r = wave * (BM / 8) + p * ROWS_PER_PASS + lane / LANES_PER_ROW;
          const v4i v = *reinterpret_cast<const v4i*>(stg + r * ROWB + ((c ^ (r & 7)) << 4));
          __builtin_amdgcn_raw_buffer_store_b128(v, ro, r * ldo + d.n0 * EB + c * 16, 0, 0);
        }
      }
    } else {
      if constexpr (!BIAS) {
        if (args.nparts > 1) {
          // split K: this part's raw fp32 sums; scale and rounding happen where the parts are added up. A lane holds
          // four consecutive features of a token per accumulator quad: one 16-byte store each.
          const int ldp = gg.n_out * 4;
          float* const pb = gg.pout + (size_t)d.part * (size_t)args.part_stride + (size_t)d.row0 * gg.n_out;
          const __amdgpu_buffer_rsrc_t rp = make_rsrc(pb, (uint32_t)d.rows_here * (uint32_t)ldp);
#pragma unroll
          for (int tt = 0; tt < TT; ++tt)
#pragma unroll
            for (int ft = 0; ft < 2; ++ft)
#pragma unroll
              for (int q = 0; q < 4; ++q) {
                v4i v;
                v.x = __float_as_int(acc[ft][tt][q * 4 + 0]);
                v.y = __float_as_int(acc[ft][tt][q * 4 + 1]);
                v.z = __float_as_int(acc[ft][tt][q * 4 + 2]);
                v.w = __float_as_int(acc[ft][tt][q * 4 + 3]);
                __builtin_amdgcn_raw_buffer_store_b128(
                    v, rp, (wt * WAVE_TOK + tt * 32 + tok32) * ldp + (d.n0 + wq * 64 + ft * 32 + q * 8 + hi32 * 4) * 4, 0, 0);
              }
          return;
        }
      }
      const float sc = ep_a;
      const int ldo = gg.n_out * 2;
      const __amdgpu_buffer_rsrc_t ro = make_rsrc(gg.out + (size_t)d.row0 * ldo, (uint32_t)d.rows_here * (uint32_t)ldo);
      // each wave stages its own 32 tokens x 64 features (128 bytes per token) at a time, two buffers in turn
      uint8_t* const mine = FP8 ? (wave < 4 ? smem + A_OFF1 + wave * 8192 : smem + B_OFF1 + (wave - 4) * 8192)
                                : stg + wave * 8192;
      const int rd_row = lane >> 3, rd_c = lane & 7;
#pragma unroll
      for (int tt = 0; tt < TT; ++tt) {
        uint8_t* const buf = mine + (tt & 1) * 4096;
        wave_sync();  // the reads of two rounds ago are ahead of these writes
#pragma unroll
        for (int ft = 0; ft < 2; ++ft) {
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            u32x2 pk;
            if constexpr (BIAS) {
              // F.linear with bias: bf16(acc + bias); then F.gelu (erf form) of that bf16 tensor, rounded again
              // (/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:14-26, 44-50). fp8: the scaled-mm epilogue
              // bf16(acc * scale_input * scale_weight + bias) of fp8_linear (/root/reference/comfy/ops.py:345-346).
              const u32x2 bq = ep_bias[ft][q];
              float v[4] = {acc[ft][tt][q * 4 + 0], acc[ft][tt][q * 4 + 1], acc[ft][tt][q * 4 + 2], acc[ft][tt][q * 4 + 3]};
              {
                // product rounded to fp32 before the bias is added (no fused multiply-add), the order the CPU
                // checker and torch's own scaled matrix multiply on the CPU use
#pragma clang fp contract(off)
                if constexpr (FP8) {
#pragma unroll
                  for (int i = 0; i < 4; ++i) v[i] = v[i] * sc;
                }
                v[0] = v[0] + Act::lo(bq.x);
                v[1] = v[1] + Act::hi(bq.x);
                v[2] = v[2] + Act::lo(bq.y);
                v[3] = v[3] + Act::hi(bq.y);
              }
              if (gg.act == 1) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                  const float h = Act::round(v[i]);
                  v[i] = 0.5f * h * (1.0f + erff(h * 0.70710678118654752440f));
                }
              }
              pk.x = Act::pack(v[0], v[1]);
              pk.y = Act::pack(v[2], v[3]);
            } else {
              pk.x = hdmoe_dev_pack_bf16(acc[ft][tt][q * 4 + 0] * sc, acc[ft][tt][q * 4 + 1] * sc);
              pk.y = hdmoe_dev_pack_bf16(acc[ft][tt][q * 4 + 2] * sc, acc[ft][tt][q * 4 + 3] * sc);
            }
            *reinterpret_cast<u32x2*>(buf + tok32 * 128 + (((ft * 4 + q) ^ (tok32 & 7)) << 4) + hi32 * 8) = pk;
          }
        }
        wave_sync();
#pragma unroll
        for (int p = 0; p < 4; ++p) {
          const int r = p * 8 + rd_row;
          const v4i v = *reinterpret_cast<const v4i*>(buf + r * 128 + ((rd_c ^ rd_row) << 4));
          __builtin_amdgcn_raw_buffer_store_b128(v, ro, (wt * WAVE_TOK + tt * 32 + r) * ldo + (d.n0 + wq * 64) * 2 + rd_c * 16, 0, 0);
        }
      }
    }
  };

  // ---- persistent loop over this block's tiles ------------------------------------------------------
  // Per tile: K steps of 128 bytes through two LDS stages, one barrier per step (the loads of step kt+1 fly
  // while step kt is multiplied). The first K step of the NEXT tile is requested before the epilogue of the
  // current one, so its latency hides behind the stores.
  Tile cur = decode(0);
  if (cur.g < 0) return;
  int gi_cur[MAX_SLABS], gi_nxt[MAX_SLABS];
#pragma unroll
  for (int j = 0; j < A_SLABS; ++j) gi_nxt[j] = -1;
  load_gather(cur, gi_cur);
  set_src(cur, gi_cur);
  kt_real = cur.nkt;
  issue_loads(0, 0);
  if constexpr (RING3) {
    if (cur.nkt > 1) issue_loads(1, 1);
  }
  for (int i = 0; cur.g >= 0; ++i) {
    const int KT = cur.nkt;
    kt_real = KT;
    load_scales(cur);
    const Tile nxt = decode(i + 1);
    if (nxt.g >= 0) load_gather(nxt, gi_nxt);  // lands during the K loop
#pragma unroll
    for (int a2 = 0; a2 < 2; ++a2)
#pragma unroll
      for (int b2 = 0; b2 < TT; ++b2)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[a2][b2][r] = 0.0f;
    // fp8: two K steps per trip, the first out of stage 0, the second out of stage 1. The barrier of a step (the
    // loads of the next step have landed for everyone, everyone has read this stage) sits between the two parts
    // of the second slice, in front of the first refill from the other stage, with TT MFMAs still to issue behind
    // it: they cover the barrier skew and the LDS latency of the first new fragments. Rows past the end of a
    // partial tile are read as zeros and multiplied like the others.
    [[maybe_unused]] auto k_loop_fp8 = [&] {
      // An odd number of steps is padded with one whose loads come from an empty buffer (zeros).
      const int KTP = (KT + 1) & ~1;
      auto sgpr = [](int v) { return __builtin_amdgcn_readfirstlane(v); };
      auto rsrc4 = [&](const v4i& r, bool real) -> v4i {  // the resource, or an empty one (every load returns zeros)
        v4i o;
        o.x = sgpr(r.x); o.y = sgpr(r.y); o.z = sgpr(real ? r.z : 0); o.w = sgpr(r.w);
        return o;
      };
      __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the first stage has landed
      __syncthreads();
      issue_loads(1, 1);                   // step 1 as a burst; from step 2 on the loads sit between the MFMAs
      fp8_fill();
      for (int kt = 0; kt < KTP; kt += 2) {
        const int more = sgpr(kt + 2 < KTP ? 1 : 0);
        // step kt out of stage 0. Its first slice requests the token rows of step kt + 1 into stage 1 (the weight
        // rows of that step went out in the second slice of step kt - 1; step 1 was requested above).
        fp8_a_loads_to1(sgpr(kt > 0 ? 1 : 0), rsrc4(ra4, kt + 1 < KT), sgpr(k_base + (kt + 1) * BK));
        fp8_b_s0k1();
        fp8_a();
        __builtin_amdgcn_s_waitcnt(0x0070);  // vmcnt(0) lgkmcnt(0): my loads of step kt + 1, my reads of stage 0
        __syncthreads();
        fp8_b_even(more, rsrc4(rb04, true), rsrc4(rb14, true), sgpr(k_base + (kt + 2) * BK));  // weights of step kt + 2 -> stage 0
        // step kt + 1 out of stage 1
        fp8_a_loads_to0(more, rsrc4(ra4, true), sgpr(k_base + (kt + 2) * BK));                 // tokens of step kt + 2 -> stage 0
        fp8_b_s1k1();
        fp8_a();
        if (more) {
          __builtin_amdgcn_s_waitcnt(0x0070);
          __syncthreads();
        }
        fp8_b_odd(more, rsrc4(rb04, kt + 3 < KT), rsrc4(rb14, kt + 3 < KT), sgpr(k_base + (kt + 3) * BK));  // weights of step kt + 3 -> stage 1
      }
    };
    [[maybe_unused]] auto k_loop = [&](auto full_c, int n_tt) {
      for (int kt = 0; kt < KT; kt += 2) {
        __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0): this wave's part of the stage has landed
        __syncthreads();                      // everyone's part has; everyone is done reading the other stage
        if (kt + 1 < KT) issue_loads(1, kt + 1);
        compute(0, full_c, n_tt);
        if (kt + 1 < KT) {
          __builtin_amdgcn_s_waitcnt(0x0f70);
          __syncthreads();
          if (kt + 2 < KT) issue_loads(0, kt + 2);
          compute(1, full_c, n_tt);
        }
      }
    };
    // Three stages: steps kt and kt + 1 are on their way when step kt is waited for (a wave's loads return in
    // order: its loads of step kt have landed when at most those of step kt + 1 are outstanding); behind the barrier
    // everyone has read stage (kt + 2) % 3, which held step kt - 1, and step kt + 2 is requested into it.
    [[maybe_unused]] auto k_loop3 = [&](auto full_c, int n_tt) {
      constexpr int PER_STEP = A_SLABS + 4;  // global->LDS loads of a wave per K step
      auto step = [&](int kt, int stage, int stage_next2) {
        // wait and barrier as one assembly statement: __syncthreads() carries a fence that waits for every
        // outstanding global->LDS load, the ones of step kt + 1 included
        if (kt + 1 < KT) asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" : : "n"(PER_STEP) : "memory");
        else asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" : : : "memory");
        if (kt + 2 < KT) issue_loads(stage_next2, kt + 2);
        compute(stage, full_c, n_tt);
      };
      for (int kt = 0; kt < KT; kt += 3) {
        step(kt, 0, 2);
        if (kt + 1 < KT) step(kt + 1, 1, 0);
        if (kt + 2 < KT) step(kt + 2, 2, 1);
      }
    };
    const int my_rows = __builtin_amdgcn_readfirstlane(cur.rows_here) - wt * WAVE_TOK;  // rows of the tile in this wave's half
    if constexpr (RING3) {
      if (my_rows > 32 * (TT - 1)) k_loop3(std::true_type{}, TT);
      else k_loop3(std::false_type{}, my_rows <= 0 ? 0 : (my_rows + 31) / 32);
    } else if constexpr (FP8 && !LIGHT) {
      k_loop_fp8();
    } else {
      if (my_rows > 32 * (TT - 1)) k_loop(std::true_type{}, TT);
      else k_loop(std::false_type{}, my_rows <= 0 ? 0 : (my_rows + 31) / 32);
    }
    // Every wave is done reading both stages: stage 0 can take the next tile's first K step, stage 1 the
    // staged outputs of this one (it is not loaded into again before the barrier of that K step).
    __syncthreads();
    if (nxt.g >= 0) {
      set_src(nxt, gi_nxt);
      kt_real = nxt.nkt;
      issue_loads(0, 0);
      if constexpr (RING3) {
        if (nxt.nkt > 1) issue_loads(1, 1);
      }
    }
    epilogue(cur);
    cur = nxt;
  }
}

// ---- split K: adding the parts up ---------------------------------------------------------------------------
// out[r, n] = bf16( (sum over parts of partial[p][r][n]) * scale(r) ), parts in ascending order (deterministic);
// scale(r) = scale_input * scale_weight of the Linear of the group that owns row r (fp8), 1 for bf16 weights.
struct SplitKReduceArgs {
  const float* partial;     // [nparts][rows_dyn + rows_static][n_out]
  long long part_stride;
  int nparts, nparts_static, n_out, rows_dyn, rows_static, n_dyn, fp8;  // parts of the dynamic rows, of the static rows
  const int32_t* offsets;   // segment bounds of the dynamic rows, n_dyn + 1 entries
  const float* sw[MAX_GROUPS];   // scale_weight per group (fp8); the static group is entry n_dyn
  const float* sin[MAX_GROUPS];  // scale_input per group or NULL
  uint16_t* out_dyn;        // [rows_dyn, n_out] bf16
  uint16_t* out_static;     // [rows_static, n_out] bf16
};

__global__ __launch_bounds__(256) void splitk_reduce_kernel(const SplitKReduceArgs a) {
  const int rows = a.rows_dyn + a.rows_static;
  const int per_row = a.n_out / 4;  // threads per row, 4 features each
  const long long total = (long long)rows * per_row;
  for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long long)gridDim.x * blockDim.x) {
    const int r = (int)(i / per_row), c = (int)(i % per_row) * 4;
    int g = a.n_dyn;  // the static group
    if (r < a.rows_dyn) {
      g = 0;
      while (g + 1 < a.n_dyn && r >= a.offsets[g + 1]) ++g;
    }
    float sc = 1.0f;
    if (a.fp8) sc = (a.sin[g] ? *a.sin[g] : 1.0f) * *a.sw[g];
    const float* src = a.partial + (size_t)r * a.n_out + c;
    float4 s = *reinterpret_cast<const float4*>(src);
    const int np = r < a.rows_dyn ? a.nparts : a.nparts_static;
    for (int p = 1; p < np; ++p) {
      const float4 t = *reinterpret_cast<const float4*>(src + (size_t)p * (size_t)a.part_stride);
      s.x += t.x; s.y += t.y; s.z += t.z; s.w += t.w;
    }
    uint2 o;
    o.x = hdmoe_dev_pack_bf16(s.x * sc, s.y * sc);
    o.y = hdmoe_dev_pack_bf16(s.z * sc, s.w * sc);
    uint16_t* dst = r < a.rows_dyn ? a.out_dyn + (size_t)r * a.n_out + c : a.out_static + (size_t)(r - a.rows_dyn) * a.n_out + c;
    *reinterpret_cast<uint2*>(dst) = o;
  }
}

template <int MODE, int TT = 4, bool LIGHT = false>
int launch_grouped(const GemmArgs& args, int tile_bound, hipStream_t s, const char* what) {
  // The opt-in for more than 64 KiB of dynamic LDS is a per-device function attribute: remembered per device
  // and instantiation (a race between two threads sets it twice, which is harmless).
  static bool attr_set[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) device = -1;
  if (device < 0 || !attr_set[device]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&grouped_gemm_kernel<MODE, TT, LIGHT>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, TileCfg<TT>::SMEM);
    if (e != hipSuccess) return hdmoe_fail(HDMOE_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    if (device >= 0) attr_set[device] = true;
  }
  if (tile_bound <= 0) return HDMOE_OK;
  // persistent blocks: one per CU (128 KiB of LDS allow no second one), a multiple of the XCD count
  int grid = (tile_bound + HDMOE_NUM_XCD - 1) / HDMOE_NUM_XCD * HDMOE_NUM_XCD;
  if (grid > HDMOE_NUM_CU) grid = HDMOE_NUM_CU;
  hipLaunchKernelGGL((grouped_gemm_kernel<MODE, TT, LIGHT>), dim3(grid), dim3(NTHREADS), TileCfg<TT>::SMEM, s, args);
  return hdmoe_check_launch(what);
}

#include "swiglu4w.h"

int launch_swiglu4w(const GemmArgs& args, int tile_bound, hipStream_t s, const char* what) {
  static bool attr_set[64] = {};
  int device = 0;
  if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) device = -1;
  if (device < 0 || !attr_set[device]) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&swiglu4w_kernel),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, W4_SMEM);
    if (e != hipSuccess) return hdmoe_fail(HDMOE_E_LAUNCH, "%s: hipFuncSetAttribute: %s", what, hipGetErrorString(e));
    if (device >= 0) attr_set[device] = true;
  }
  if (tile_bound <= 0) return HDMOE_OK;
  int grid = (tile_bound + HDMOE_NUM_XCD - 1) / HDMOE_NUM_XCD * HDMOE_NUM_XCD;
  if (grid > HDMOE_NUM_CU) grid = HDMOE_NUM_CU;
  hipLaunchKernelGGL(swiglu4w_kernel, dim3(grid), dim3(W4_THREADS), W4_SMEM, s, args);
  return hdmoe_check_launch(what);
}

inline int elem_bytes(int weight_dtype) { return weight_dtype == HDMOE_W_E4M3FN ? 1 : 2; }

int check_dtype(int weight_dtype, const char* what) {
  if (weight_dtype != HDMOE_W_BF16 && weight_dtype != HDMOE_W_E4M3FN)
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: weight_dtype=%d is neither HDMOE_W_BF16 nor HDMOE_W_E4M3FN", what, weight_dtype);
  return HDMOE_OK;
}

}  // namespace

// ---- which kernel runs a feed-forward contraction ---------------------------------------------------------------
// Two process-wide switches choose between kernels with the same results bit for bit (hdmoe_set_kernel_form). Their
// initial values come from the environment variables HDMOE_SWIGLU4W / HDMOE_LIGHT, read once ("0" = never, anything
// else = always, unset = the launcher's own rule).
namespace {
std::atomic<int> g_form[HDMOE_NUM_FORMS] = {{HDMOE_FORM_AUTO}, {HDMOE_FORM_AUTO}};
std::once_flag g_form_once;
void form_init() {
  static const char* const names[HDMOE_NUM_FORMS] = {"HDMOE_SWIGLU4W", "HDMOE_LIGHT"};
  for (int i = 0; i < HDMOE_NUM_FORMS; ++i) {
    const char* v = getenv(names[i]);
    if (v != nullptr) g_form[i].store(v[0] == '0' ? HDMOE_FORM_NEVER : HDMOE_FORM_ALWAYS, std::memory_order_relaxed);
  }
}
int form_of(int which) {
  std::call_once(g_form_once, form_init);
  return g_form[which].load(std::memory_order_relaxed);
}

// The kernels a contraction of the feed-forward can run on.
enum GemmForm {
  FORM_SPLIT_K,    // plain modes cut along K (few tiles); its own choice of tile inside
  FORM_RING3,      // 128-token tiles, three LDS stages, token blocks without rows skipped
  FORM_LIGHT4,     // 256-token tiles, token blocks without rows skipped
  FORM_W4,         // fp8 gate/up: the 4-wave kernel (256-token tiles)
  FORM_TALL5,      // 320-token tiles
  FORM_BASE4       // 256-token tiles
};

struct GemmShape {
  bool swiglu, fp8, split;
  int rows_dyn, n_dyn, rows_static;  // rows_static = 0: no static group
  int N_dyn, N_static;
  bool w4_fits;                      // the 4-wave kernel takes these operands (swiglu4w_fits)
};

// Expected tiles with evenly loaded experts, static round-robin over the CUs, and a fixed cost per tile of about one
// 32-token block: rounds x (TT + 1). The taller tile wins when it does not add a round.
long expected_tile_cost(const GemmShape& sh, int tt) {
  const int bm = 64 * tt, fpt = sh.swiglu ? BN / 2 : BN;
  long tiles = 0;
  if (sh.n_dyn > 0) tiles += (long)sh.n_dyn * ((sh.rows_dyn / sh.n_dyn + bm - 1) / bm) * (sh.N_dyn / fpt);
  if (sh.rows_static > 0) tiles += (long)((sh.rows_static + bm - 1) / bm) * (sh.N_static / fpt);
  return ((tiles + HDMOE_NUM_CU - 1) / HDMOE_NUM_CU) * (tt + 1);
}

// light: the token blocks of a tile that hold no rows are skipped (fp8: the compiler-scheduled K loop instead of the
// assembly loop, which multiplies padding like rows; 16-bit weights always skip them and take from this only the
// three-stage ring).
struct FormChoice { GemmForm form; bool light, ring16, tall; };
FormChoice pick_form(const GemmShape& sh) {
  const int f_light = form_of(HDMOE_FORM_LIGHT), f_4w = form_of(HDMOE_FORM_SWIGLU4W);
  const bool few_rows = hdmoe_few_rows(sh.rows_dyn, sh.n_dyn, sh.rows_static);
  FormChoice c;
  // forcing the 4-wave kernel also keeps the light form's default off
  c.light = sh.fp8 && (f_light != HDMOE_FORM_AUTO ? f_light == HDMOE_FORM_ALWAYS
                                                   : few_rows && !(sh.swiglu && f_4w == HDMOE_FORM_ALWAYS));
  c.ring16 = !sh.fp8 && few_rows && f_light != HDMOE_FORM_NEVER;
  // (bf16: the gate/up kernel only; the down projection measured slower on the taller tile)
  c.tall = (sh.fp8 || sh.swiglu) && !sh.split && !c.light && expected_tile_cost(sh, 5) < expected_tile_cost(sh, 4);
  if (sh.split) { c.form = FORM_SPLIT_K; return c; }
  // Light form, gate/up: with every segment inside one 128-token tile (up to 128 tokens in a top-2 layer of 4 experts)
  // the three-stage ring of the down projection pays here too (whole layer 78 -> 73 us at 16 tokens, 80 -> 75 at 128;
  // at 256 tokens the shared expert's second m-tile costs more than the ring gains: 93 -> 105 us).
  if ((c.light || c.ring16) && sh.swiglu && sh.rows_static <= TileCfg<2>::BM &&
      (sh.n_dyn <= 0 || sh.rows_dyn <= TileCfg<2>::BM / 2 * sh.n_dyn)) {
    c.form = FORM_RING3;
    return c;
  }
  if (c.light) { c.form = FORM_LIGHT4; return c; }
  // The 4-wave form of the gate/up kernel (swiglu4w.h) has the 256-token tile; it takes the launch whenever the
  // 8-wave kernel would not use its 320-token tile (2-3 % faster there: part of its epilogue hides in the K loop).
  const bool want4w = f_4w != HDMOE_FORM_AUTO ? f_4w == HDMOE_FORM_ALWAYS : !c.tall;
  if (sh.fp8 && sh.swiglu && want4w && sh.w4_fits) { c.form = FORM_W4; return c; }
  c.form = c.tall ? FORM_TALL5 : FORM_BASE4;
  return c;
}
}  // namespace

extern "C" int hdmoe_set_kernel_form(int which, int value) {
  if (which < 0 || which >= HDMOE_NUM_FORMS || value < HDMOE_FORM_AUTO || value > HDMOE_FORM_ALWAYS)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_set_kernel_form: which=%d value=%d", which, value);
  std::call_once(g_form_once, form_init);
  g_form[which].store(value, std::memory_order_relaxed);
  return HDMOE_OK;
}

extern "C" int hdmoe_get_kernel_form(int which) {
  if (which < 0 || which >= HDMOE_NUM_FORMS) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_get_kernel_form: which=%d", which);
  return form_of(which);
}

// Shared by hdmoe_grouped_swiglu / hdmoe_grouped_down / hdmoe_linear / hdmoe_moe_ffn.
// groups: n_dyn experts with device-side segments, optionally one static group (the shared expert).
// gather_dyn (optional): the routed rows are not materialised in segment order; row r of the segments is row
// gather_dyn[r] of a_dyn, which holds gather_rows rows.
int hdmoe_launch_ffn_gemm(bool swiglu, int weight_dtype, const uint8_t* a_dyn, const int32_t* offsets, int rows_dyn,
                          int n_dyn, const hdmoe_ffn_weights* experts, uint8_t* out_dyn, const uint8_t* a_static,
                          int rows_static, const hdmoe_ffn_weights* shared, uint8_t* out_static, int K_dyn, int N_dyn,
                          int K_static, int N_static, hipStream_t s, const char* what,
                          const int32_t* gather_dyn = nullptr, int gather_rows = 0, float* partial = nullptr,
                          int nparts = 1, int gather_shift = 0, bool reduce = true,
                          const HdmoeSplitPlan* plan = nullptr, const HdmoeAltOperand* alt = nullptr) {
  const int eb = elem_bytes(weight_dtype);
  const bool fp8 = weight_dtype == HDMOE_W_E4M3FN;
  const int feat_per_tile = swiglu ? BN / 2 : BN;
  // Split K (runs on the 256-token tile, or the 128-token one of the light form): nparts = the most parts any entry of
  // the plan cuts a tile into (the partial-sum buffer holds that many); no plan = every tile in nparts parts
  const bool split = !swiglu && partial != nullptr && nparts > 1;
  GemmShape shape;
  shape.swiglu = swiglu; shape.fp8 = fp8; shape.split = split;
  shape.rows_dyn = rows_dyn; shape.n_dyn = n_dyn; shape.rows_static = shared != nullptr ? rows_static : 0;
  shape.N_dyn = N_dyn; shape.N_static = N_static;
  shape.w4_fits = true;  // settled below, once the groups are filled in
  FormChoice choice = pick_form(shape);
  const bool light = choice.light, ring16 = choice.ring16, tall = choice.tall;
  const int BM = tall ? TileCfg<5>::BM : TileCfg<4>::BM;  // tokens per block tile of the kernel that will run
  const int gather_rows_max = (alt != nullptr && alt->rows > gather_rows) ? alt->rows : gather_rows;
  if (gather_dyn != nullptr && (unsigned long long)gather_rows_max * K_dyn * eb >= (1ull << 31))
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: %d gathered rows of %d bytes exceed the 2 GiB offset range", what,
                      gather_rows_max, K_dyn * eb);
  GemmArgs args;
  memset(&args, 0, sizeof(args));
  if (alt != nullptr && gather_dyn != nullptr) args.alt = *alt;
  args.nparts = 1;
  args.offsets = offsets;
  args.n_offsets = n_dyn;
  int G = 0, tile_bound = 0;
  for (int e = 0; e < n_dyn; ++e, ++G) {
    GemmGroup& gg = args.g[G];
    const hdmoe_ffn_weights& w = experts[e];
    gg.a = a_dyn;
    gg.gather = gather_dyn;
    gg.gather_shift = gather_shift;
    gg.a_rows = gather_rows;
    gg.out = out_dyn;
    gg.row_begin = -1;
    gg.dyn = e;
    gg.n_out = N_dyn;
    gg.kbytes = K_dyn * eb;
    if (swiglu) {
      gg.b0 = static_cast<const uint8_t*>(w.w1); gg.b1 = static_cast<const uint8_t*>(w.w3);
      gg.sb0 = w.scale_w1; gg.sb1 = w.scale_w3; gg.s_in = w.scale_in1; gg.s_in_b = w.scale_in3; gg.s_next = w.scale_in2;
    } else {
      gg.b0 = static_cast<const uint8_t*>(w.w2); gg.sb0 = w.scale_w2; gg.s_in = w.scale_in2;
    }
    if (!gg.b0 || (swiglu && !gg.b1)) return hdmoe_fail(HDMOE_E_NULL, "%s: expert %d has a NULL weight", what, e);
    if (fp8 && (!gg.sb0 || (swiglu && !gg.sb1)))
      return hdmoe_fail(HDMOE_E_NULL, "%s: expert %d has a NULL scale_weight", what, e);
  }
  int tb_dyn = 0, tb_static = 0;  // the two summands of tile_bound
  if (n_dyn > 0) tb_dyn = (rows_dyn / BM + n_dyn) * (N_dyn / feat_per_tile);
  tile_bound += tb_dyn;
  if (shared != nullptr && rows_static > 0) {
    GemmGroup& gg = args.g[G];
    const hdmoe_ffn_weights& w = *shared;
    gg.a = a_static;
    gg.out = out_static;
    gg.row_begin = 0;
    gg.row_end = rows_static;
    gg.n_out = N_static;
    gg.kbytes = K_static * eb;
    if (swiglu) {
      gg.b0 = static_cast<const uint8_t*>(w.w1); gg.b1 = static_cast<const uint8_t*>(w.w3);
      gg.sb0 = w.scale_w1; gg.sb1 = w.scale_w3; gg.s_in = w.scale_in1; gg.s_in_b = w.scale_in3; gg.s_next = w.scale_in2;
    } else {
      gg.b0 = static_cast<const uint8_t*>(w.w2); gg.sb0 = w.scale_w2; gg.s_in = w.scale_in2;
    }
    if (!gg.b0 || (swiglu && !gg.b1)) return hdmoe_fail(HDMOE_E_NULL, "%s: static group has a NULL weight", what);
    if (fp8 && (!gg.sb0 || (swiglu && !gg.sb1)))
      return hdmoe_fail(HDMOE_E_NULL, "%s: static group has a NULL scale_weight", what);
    tb_static = ((rows_static + BM - 1) / BM) * (N_static / feat_per_tile);
    tile_bound += tb_static;
    ++G;
  }
  args.G = G;
  // tiles of the static group are shorter or longer than the experts' when the two K differ (down projection)
  if (n_dyn > 0 && shared != nullptr && rows_static > 0 && K_static != K_dyn) args.spread = K_static < K_dyn ? 1 : -1;
  if (split) {
    // fp32 partial sums [nparts][rows_dyn + rows_static][N] (N_dyn == N_static is required), then the kernel that
    // adds them up, applies the scales and rounds to bf16
    if (n_dyn > 0 && shared != nullptr && rows_static > 0 && N_dyn != N_static)
      return hdmoe_fail(HDMOE_E_SHAPE, "%s: split K needs one output width, got %d and %d", what, N_dyn, N_static);
    const int N = n_dyn > 0 ? N_dyn : N_static;
    const int rows_all = (n_dyn > 0 ? rows_dyn : 0) + ((shared != nullptr && rows_static > 0) ? rows_static : 0);
    args.nparts = nparts;  // > 1: every group leaves fp32 sums
    args.part_stride = (long long)rows_all * N;
    for (int g = 0; g < G; ++g)
      args.g[g].pout = partial + (args.g[g].row_begin < 0 ? 0 : (size_t)(n_dyn > 0 ? rows_dyn : 0) * N);
    constexpr int BM2 = TileCfg<2>::BM;
    if (plan != nullptr && plan->n >= 1 && plan->n <= HDMOE_PLAN_MAX && plan->bm > 0) {
      args.plan = *plan;  // as the caller's other kernel sees it, tile height and limit included
    } else {
      args.plan.n = 1;
      args.plan.pd[0] = args.plan.ps[0] = nparts;
      args.plan.bm = (light || ring16) ? BM2 : BM;
      args.plan.max_tiles = HDMOE_NUM_CU;
    }
    if (reduce && args.plan.n > 1) {  // splitk_reduce_kernel takes a fixed cut: the plan's last entry
      args.plan.pd[0] = args.plan.pd[args.plan.n - 1];
      args.plan.ps[0] = args.plan.ps[args.plan.n - 1];
      args.plan.n = 1;
    }
    for (int i = 0; i < args.plan.n; ++i)
      if (args.plan.pd[i] < 1 || args.plan.pd[i] > nparts || args.plan.ps[i] < 1 || args.plan.ps[i] > nparts)
        return hdmoe_fail(HDMOE_E_SHAPE, "%s: split plan entry %d cuts in %d / %d parts, buffer holds %d", what, i,
                          args.plan.pd[i], args.plan.ps[i], nparts);
    // grid: enough blocks for the entry with the most tiles
    int tb_light = 0;  // the light form cut along K runs on 128-token tiles with a three-stage ring
    tile_bound = 0;
    for (int i = 0; i < args.plan.n; ++i) {
      const int tb = tb_dyn * args.plan.pd[i] + tb_static * args.plan.ps[i];
      if (tb > tile_bound) tile_bound = tb;
      if (light || ring16) {
        int tl = 0;
        if (n_dyn > 0) tl += (rows_dyn / BM2 + n_dyn) * (N_dyn / feat_per_tile) * args.plan.pd[i];
        if (shared != nullptr && rows_static > 0)
          tl += ((rows_static + BM2 - 1) / BM2) * (N_static / feat_per_tile) * args.plan.ps[i];
        if (tl > tb_light) tb_light = tl;
      }
    }
    const int rc = light ? launch_grouped<FP8_PLAIN, 2, true>(args, tb_light, s, what)
                   : ring16 ? launch_grouped<BF16_PLAIN, 2, true>(args, tb_light, s, what)
                   : fp8 ? launch_grouped<FP8_PLAIN>(args, tile_bound, s, what)
                         : launch_grouped<BF16_PLAIN>(args, tile_bound, s, what);
    if (rc != HDMOE_OK) return rc;
    if (!reduce) return HDMOE_OK;  // the caller's next kernel adds the parts up (hdmoe_launch_combine_partials)
    SplitKReduceArgs ra;
    memset(&ra, 0, sizeof(ra));
    ra.partial = partial;
    ra.part_stride = args.part_stride;
    ra.nparts = args.plan.pd[0];
    ra.nparts_static = args.plan.ps[0];
    ra.n_out = N;
    ra.rows_dyn = n_dyn > 0 ? rows_dyn : 0;
    ra.rows_static = (shared != nullptr && rows_static > 0) ? rows_static : 0;
    ra.n_dyn = n_dyn;
    ra.fp8 = fp8 ? 1 : 0;
    ra.offsets = offsets;
    for (int g = 0; g < G; ++g) {
      const int slot = args.g[g].row_begin < 0 ? args.g[g].dyn : n_dyn;
      ra.sw[slot] = args.g[g].sb0;
      ra.sin[slot] = args.g[g].s_in;
    }
    ra.out_dyn = reinterpret_cast<uint16_t*>(out_dyn);
    ra.out_static = reinterpret_cast<uint16_t*>(out_static);
    const long long work = (long long)rows_all * (N / 4);
    int blocks = (int)((work + 255) / 256);
    if (blocks > HDMOE_NUM_CU * 8) blocks = HDMOE_NUM_CU * 8;
    if (blocks < 1) blocks = 1;
    hipLaunchKernelGGL(splitk_reduce_kernel, dim3(blocks), dim3(256), 0, s, ra);
    return hdmoe_check_launch(what);
  }
  if (fp8 && swiglu) {
    long long op_bytes = (long long)(gather_dyn != nullptr ? gather_rows_max : rows_dyn) * K_dyn;
    if ((long long)rows_static * K_static > op_bytes) op_bytes = (long long)rows_static * K_static;
    shape.w4_fits = swiglu4w_fits(args, op_bytes);
    choice = pick_form(shape);
  }
  switch (choice.form) {
    case FORM_RING3: {
      constexpr int BM2 = TileCfg<2>::BM;
      int tb = 0;
      if (n_dyn > 0) tb += (rows_dyn / BM2 + n_dyn) * (N_dyn / feat_per_tile);
      if (shared != nullptr && rows_static > 0) tb += ((rows_static + BM2 - 1) / BM2) * (N_static / feat_per_tile);
      return fp8 ? launch_grouped<FP8_SWIGLU, 2, true>(args, tb, s, what)
                 : launch_grouped<BF16_SWIGLU, 2, true>(args, tb, s, what);
    }
    case FORM_LIGHT4:
      return swiglu ? launch_grouped<FP8_SWIGLU, 4, true>(args, tile_bound, s, what)
                    : launch_grouped<FP8_PLAIN, 4, true>(args, tile_bound, s, what);
    case FORM_W4: {
      int tb = 0;
      if (n_dyn > 0) tb += (rows_dyn / W4_BM + n_dyn) * (N_dyn / W4_FEAT);
      if (shared != nullptr && rows_static > 0) tb += ((rows_static + W4_BM - 1) / W4_BM) * (N_static / W4_FEAT);
      return launch_swiglu4w(args, tb, s, what);
    }
    case FORM_TALL5:
      if (fp8) return swiglu ? launch_grouped<FP8_SWIGLU, 5>(args, tile_bound, s, what)
                             : launch_grouped<FP8_PLAIN, 5>(args, tile_bound, s, what);
      return launch_grouped<BF16_SWIGLU, 5>(args, tile_bound, s, what);
    default:
      break;
  }
  if (fp8) return swiglu ? launch_grouped<FP8_SWIGLU>(args, tile_bound, s, what)
                         : launch_grouped<FP8_PLAIN>(args, tile_bound, s, what);
  return swiglu ? launch_grouped<BF16_SWIGLU>(args, tile_bound, s, what)
                : launch_grouped<BF16_PLAIN>(args, tile_bound, s, what);
}

// Name of the kernel the gate/up contraction of a layer runs on (T tokens, E routed experts top-2 plus a shared expert
// if Hs > 0), by the launcher's own rule and the current form switches: for reports that name the dominant kernel.
extern "C" const char* hdmoe_gate_up_kernel_name(int weight_dtype, int T, int E, int D, int H, int Hs,
                                                 int has_scale_in2) {
  if (check_dtype(weight_dtype, "hdmoe_gate_up_kernel_name") != HDMOE_OK || T <= 0 || E < 0 || D <= 0 || H <= 0)
    return "";
  GemmShape sh;
  sh.swiglu = true; sh.fp8 = weight_dtype == HDMOE_W_E4M3FN; sh.split = false;
  sh.rows_dyn = E > 0 ? T * HDMOE_TOPK : 0; sh.n_dyn = E; sh.rows_static = Hs > 0 ? T : 0;
  sh.N_dyn = H; sh.N_static = Hs;
  const int kb = D * elem_bytes(weight_dtype);
  sh.w4_fits = sh.fp8 && has_scale_in2 != 0 && kb % (2 * BK) == 0 && kb >= 16 * BK && H % W4_FEAT == 0 &&
               (Hs <= 0 || Hs % W4_FEAT == 0) && (long long)T * kb < (1ll << 31);
  switch (pick_form(sh).form) {
    case FORM_RING3: return sh.fp8 ? "grouped_gemm_kernel<FP8_SWIGLU, 2, LIGHT>" : "grouped_gemm_kernel<BF16_SWIGLU, 2, LIGHT>";
    case FORM_LIGHT4: return "grouped_gemm_kernel<FP8_SWIGLU, 4, LIGHT>";
    case FORM_W4: return "swiglu4w_kernel";
    case FORM_TALL5: return sh.fp8 ? "grouped_gemm_kernel<FP8_SWIGLU, 5>" : "grouped_gemm_kernel<BF16_SWIGLU, 5>";
    default: return sh.fp8 ? "grouped_gemm_kernel<FP8_SWIGLU, 4>" : "grouped_gemm_kernel<BF16_SWIGLU, 4>";
  }
}

// How the down projection of a layer is cut along K: a pure function of the sizes, so that the workspace layout and
// the launch agree. With few tiles (small token counts) most CUs would idle through a long K loop. Returns the most
// parts any entry of the plan cuts a tile into (the partial-sum buffer is sized for it; 1 = no cut) and fills *plan.
//
// Cost model in units of one K step of one tile: a tile costs its steps + 3 (prologue and epilogue); one round of
// blocks lasts as long as its longest tile; more tiles than CUs last about the total divided by the CUs plus half a
// tile of slack; a cut adds the fp32 partial sums written and read again (8 bytes per output and part; they stay in
// the memory-side cache at these sizes, about 10 TB/s; one step is about 1.4 us).
int hdmoe_down_parts(int rows_dyn, int n_dyn, int rows_static, int N, int K_dyn, int K_static, int weight_dtype,
                     HdmoeSplitPlan* plan) {
  HdmoeSplitPlan local;
  HdmoeSplitPlan& pl = plan != nullptr ? *plan : local;
  memset(&pl, 0, sizeof(pl));
  pl.bm = TileCfg<4>::BM;
  pl.max_tiles = HDMOE_NUM_CU;
  auto fixed = [&](int parts) {
    pl.n = 1;
    pl.pd[0] = pl.ps[0] = parts;
    return parts;
  };
  const int eb = elem_bytes(weight_dtype);
  const int nt = N / BN;
  const bool dyn = n_dyn > 0 && rows_dyn > 0;
  const int ktd = dyn ? K_dyn * eb / BK : 0, kts = rows_static > 0 ? K_static * eb / BK : 0;
  if ((!dyn && rows_static <= 0) || nt <= 0 || (ktd <= 0 && kts <= 0)) return fixed(1);

  // Few rows per segment (the rule of the light form in hdmoe_launch_ffn_gemm): the launch runs on 128-token
  // tiles with K steps requested two ahead, and is bound by how fast the weights arrive, not by its K loops. About 150
  // blocks keep enough loads in flight; more parts only add partial sums. The mean segment sits near the tile height,
  // so segments are counted 1.5 times the mean: an expert that needs a second m-tile must not push the launch into a
  // second round of blocks. (Whole layer, uniform / skewed routing, 256 tokens: 2 parts 99 / 102 us, 3 parts 95 / 110
  // us; 128 tokens: 2 parts 88, 3 parts 81, 5 parts 96 us.)
  if (hdmoe_few_rows(rows_dyn, n_dyn, rows_static)) {
    const int bm2 = TileCfg<2>::BM;
    pl.bm = bm2;
    long t2 = 0;
    if (dyn) {
      const long seg = ((long)rows_dyn * 3 / 2 + n_dyn - 1) / n_dyn;
      t2 += (long)n_dyn * ((seg + bm2 - 1) / bm2) * nt;
    }
    if (rows_static > 0) t2 += (long)((rows_static + bm2 - 1) / bm2) * nt;
    const int kt2 = ktd > kts ? ktd : kts;
    long parts = (150 + t2 - 1) / t2;
    if (parts > HDMOE_NUM_CU / t2) parts = HDMOE_NUM_CU / t2;
    if (parts > 6) parts = 6;
    while (parts > 1 && kt2 / parts < 6) --parts;
    return fixed(parts < 1 ? 1 : (int)parts);
  }

  const int bm = TileCfg<4>::BM;
  const double red_unit = (double)N * 8.0 / 10e12 / 1.4e-6;  // K steps per row and part of partial sums
  if (!dyn || rows_static <= 0) {
    // one kind of group: every tile in the same number of parts, whole rounds of tiles
    double tiles = 0;
    if (dyn) tiles += 1.12 * n_dyn * ((rows_dyn / n_dyn + bm - 1) / bm) * nt;
    if (rows_static > 0) tiles += (double)((rows_static + bm - 1) / bm) * nt;
    const int kt = ktd > kts ? ktd : kts;
    const double rows_all = (double)(dyn ? rows_dyn : 0) + (rows_static > 0 ? rows_static : 0);
    int best = 1;
    double best_cost = 0;
    for (int parts = 1; parts <= 6 && kt / parts >= 6; ++parts) {
      const double rounds = (double)(long)((tiles * parts + HDMOE_NUM_CU - 1) / HDMOE_NUM_CU);
      const double cost = rounds * ((double)kt / parts + 3.0) + (parts > 1 ? parts * rows_all * red_unit : 0.0);
      if (parts == 1 || cost < best_cost * 0.95) {  // a cut has to pay
        best = parts;
        best_cost = cost;
      }
    }
    return fixed(best);
  }

  // Experts and a static group (the layer). Their tiles have different K (HiDream: 6912 and 3584), and cutting the
  // static group's tiles in ps = pd * kts / ktd parts makes all tiles about equally long.
  // Candidates, most parts first, every tile alike before the equalising cut: the cuts whose tiles fit one round of
  // blocks with every expert at the mean segment size. The device takes the first that really fits (measured on 4
  // experts + shared expert, fp8 and bf16: 320-384 tokens (4,4) or (4,2), 512 tokens (3,3) or (3,2), 640-896 tokens
  // (2,2) or (2,1), 1024 tokens (2,1), each 2-10 % ahead of any cut that needs a second round).
  const int mt_d_mean = n_dyn * ((rows_dyn / n_dyn + bm - 1) / bm), mt_s = (rows_static + bm - 1) / bm;
  pl.n = 0;
  auto candidate = [&](int pd, int ps) {
    if (pl.n >= HDMOE_PLAN_MAX - 1 || (mt_d_mean * pd + mt_s * ps) * nt > HDMOE_NUM_CU) return;
    for (int i = 0; i < pl.n; ++i)
      if (pl.pd[i] == pd && pl.ps[i] == ps) return;
    pl.pd[pl.n] = pd;
    pl.ps[pl.n] = ps;
    ++pl.n;
  };
  for (int pd = 6; pd >= 2; --pd) {
    if (ktd / pd < 6) continue;
    int ps = (int)((double)pd * kts / ktd + 0.5);
    if (ps < 1) ps = 1;
    if (ps > pd) ps = pd;
    while (ps > 1 && kts / ps < 6) --ps;
    if (kts / pd >= 6) candidate(pd, pd);
    candidate(pd, ps);
  }
  // A first candidate that still fits with every expert one standard deviation above the mean segment (the counts
  // are about binomial) is taken as it is: the kernels then have nothing to decide (the decision costs them about a
  // microsecond each).
  const double mu = (double)rows_dyn / n_dyn;
  if (pl.n > 0) {
    const int mt_d_hi = n_dyn * (int)(((long)(mu + sqrt(mu)) + bm - 1) / bm);
    if ((mt_d_hi * pl.pd[0] + mt_s * pl.ps[0]) * nt <= HDMOE_NUM_CU) {
      pl.n = 1;
      return pl.pd[0];
    }
  }
  // Last entry, for when no candidate fits: the cheapest cut by the cost model. With candidates listed, their not
  // fitting means ragged segments, and the experts' m-tiles are counted one standard deviation above the mean
  // segment (counts are about binomial); with none, 12 % above the mean.
  const double seg = pl.n > 0 ? mu + sqrt(mu) : mu;
  const double td = (pl.n > 0 ? 1.0 : 1.12) * n_dyn * (double)(((long)seg + bm - 1) / bm) * nt, ts = (double)mt_s * nt;
  int best_d = 1, best_s = 1;
  double best_cost = 0;
  for (int pd = 1; pd <= 6 && (pd == 1 || ktd / pd >= 6); ++pd)
    for (int ps = 1; ps <= pd && (ps == 1 || kts / ps >= 6); ++ps) {
      const double ld = (double)ktd / pd + 3.0, ls = (double)kts / ps + 3.0;
      const double tiles = td * pd + ts * ps, longest = ld > ls ? ld : ls;
      double cost = tiles <= HDMOE_NUM_CU ? longest : (td * pd * ld + ts * ps * ls) / HDMOE_NUM_CU + 0.5 * longest;
      if (pd > 1) cost += ((double)rows_dyn * pd + (double)rows_static * ps) * red_unit;
      if ((pd == 1 && ps == 1) || cost < best_cost * 0.95) {
        best_d = pd;
        best_s = pd > 1 ? ps : 1;
        best_cost = cost;
      }
    }
  pl.pd[pl.n] = best_d;
  pl.ps[pl.n] = best_s;
  ++pl.n;
  int most = 1;
  for (int i = 0; i < pl.n; ++i) most = pl.pd[i] > most ? pl.pd[i] : most;
  if (most == 1) return fixed(1);  // nothing is cut
  return most;
}

// Linear with bias and optional GELU over expert row segments plus an optional static group (bf16 weights):
// the two stages of a GELU feed-forward (/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:28-50, 114-188).
int hdmoe_launch_linear_groups(const uint8_t* a_dyn, const int32_t* offsets, int rows_dyn, int n_dyn,
                               const hdmoe_linear_weights* experts, uint8_t* out_dyn, const uint8_t* a_static,
                               int rows_static, const hdmoe_linear_weights* shared, uint8_t* out_static, int K, int N,
                               int act, hipStream_t s, const char* what, bool f16 = false,
                               const int32_t* gather = nullptr, int gather_rows = 0, int gather_shift = 0) {
  if (gather != nullptr && (unsigned long long)gather_rows * K * 2 >= (1ull << 31))
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: %d gathered rows of %d bytes exceed the 2 GiB offset range", what, gather_rows,
                      K * 2);
  GemmArgs args;
  memset(&args, 0, sizeof(args));
  args.nparts = 1;
  args.offsets = offsets;
  args.n_offsets = n_dyn;
  int G = 0, tile_bound = 0;
  auto fill = [&](GemmGroup& gg, const hdmoe_linear_weights& w) {
    gg.b0 = static_cast<const uint8_t*>(w.weight);
    gg.bias = static_cast<const uint16_t*>(w.bias);
    gg.act = act;
    gg.n_out = N;
    gg.kbytes = K * 2;
  };
  for (int e = 0; e < n_dyn; ++e, ++G) {
    GemmGroup& gg = args.g[G];
    fill(gg, experts[e]);
    gg.a = a_dyn;
    gg.gather = gather;
    gg.gather_shift = gather_shift;
    gg.a_rows = gather_rows;
    gg.out = out_dyn;
    gg.row_begin = -1;
    gg.dyn = e;
    if (!gg.b0) return hdmoe_fail(HDMOE_E_NULL, "%s: expert %d has a NULL weight", what, e);
  }
  // tile height by the rule of the feed-forward GEMMs: the 320-token tile when it saves a round of tiles
  auto expected_cost = [&](int tt) {
    const int bm = 64 * tt;
    long tiles = 0;
    // a segment taken one standard deviation of an even routing above the mean: at a mean that is a multiple of the
    // tile height half the segments need one tile more
    const int seg = n_dyn > 0 ? rows_dyn / n_dyn + (int)sqrtf((float)(rows_dyn / n_dyn)) : 0;
    if (n_dyn > 0) tiles += (long)n_dyn * ((seg + bm - 1) / bm) * (N / BN);
    if (shared != nullptr && rows_static > 0) tiles += (long)((rows_static + bm - 1) / bm) * (N / BN);
    return ((tiles + HDMOE_NUM_CU - 1) / HDMOE_NUM_CU) * (tt + 1);
  };
  const bool tall = expected_cost(5) < expected_cost(4);
  const int BM = tall ? TileCfg<5>::BM : TileCfg<4>::BM;
  if (n_dyn > 0) tile_bound += (rows_dyn / BM + n_dyn) * (N / BN);
  if (shared != nullptr && rows_static > 0) {
    GemmGroup& gg = args.g[G];
    fill(gg, *shared);
    gg.a = a_static;
    gg.out = out_static;
    gg.row_begin = 0;
    gg.row_end = rows_static;
    if (!gg.b0) return hdmoe_fail(HDMOE_E_NULL, "%s: static group has a NULL weight", what);
    tile_bound += ((rows_static + BM - 1) / BM) * (N / BN);
    ++G;
  }
  args.G = G;
  if (tall) return f16 ? launch_grouped<F16_PLAIN_BIAS, 5>(args, tile_bound, s, what)
                       : launch_grouped<BF16_PLAIN_BIAS, 5>(args, tile_bound, s, what);
  return f16 ? launch_grouped<F16_PLAIN_BIAS>(args, tile_bound, s, what)
             : launch_grouped<BF16_PLAIN_BIAS>(args, tile_bound, s, what);
}

// One Linear with an optional bias over all rows of `a` (either weight type): a single static group.
int hdmoe_launch_linear_bias(int weight_dtype, const uint8_t* a, int rows, int K, int N, const uint8_t* w,
                             const float* scale_w, const float* scale_in, const uint16_t* bias, uint8_t* out,
                             hipStream_t s, const char* what) {
  const bool fp8 = weight_dtype == HDMOE_W_E4M3FN;
  GemmArgs args;
  memset(&args, 0, sizeof(args));
  args.nparts = 1;
  GemmGroup& gg = args.g[0];
  gg.a = a;
  gg.out = out;
  gg.row_begin = 0;
  gg.row_end = rows;
  gg.n_out = N;
  gg.kbytes = K * elem_bytes(weight_dtype);
  gg.b0 = w;
  gg.sb0 = scale_w;
  gg.s_in = scale_in;
  gg.bias = bias;
  gg.act = HDMOE_ACT_NONE;
  args.G = 1;
  const int tile_bound = ((rows + TileCfg<4>::BM - 1) / TileCfg<4>::BM) * (N / BN);
  if (weight_dtype == HDMOE_W_F16) return launch_grouped<F16_PLAIN_BIAS>(args, tile_bound, s, what);
  return fp8 ? launch_grouped<FP8_PLAIN_BIAS>(args, tile_bound, s, what)
             : launch_grouped<BF16_PLAIN_BIAS>(args, tile_bound, s, what);
}

// Size rules shared by the entry points: K bytes per row must be a multiple of the
// 128-byte K step; total bytes of each operand must fit the 32-bit buffer range.
int hdmoe_check_gemm_shape(const char* what, int weight_dtype, long rows, int K, int N, int feat_per_tile) {
  if (int rc = check_dtype(weight_dtype, what)) return rc;
  const int eb = elem_bytes(weight_dtype);
  if (rows < 0 || K <= 0 || N <= 0 || (K * eb) % BK != 0 || N % feat_per_tile != 0)
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: rows=%ld K=%d N=%d (K*%d must be a multiple of %d, N of %d)", what, rows, K,
                      N, eb, BK, feat_per_tile);
  if ((unsigned long long)rows * K * eb >= (1ull << 32) || (unsigned long long)rows * N * 2 >= (1ull << 40))
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: rows=%ld K=%d exceeds the 4 GiB buffer range", what, rows, K);
  return HDMOE_OK;
}

extern "C" int hdmoe_grouped_swiglu(int weight_dtype, const void* a, const int32_t* offsets, int rows_total, int E,
                                    int D, int H, const hdmoe_ffn_weights* experts, void* h, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(a);
  HDMOE_REQUIRE_PTR(offsets);
  HDMOE_REQUIRE_PTR(experts);
  HDMOE_REQUIRE_PTR(h);
  if (E < 1 || E > HDMOE_MAX_EXPERTS) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_grouped_swiglu: E=%d", E);
  if (int rc = hdmoe_check_gemm_shape("hdmoe_grouped_swiglu", weight_dtype, rows_total, D, H, BN / 2)) return rc;
  if (weight_dtype == HDMOE_W_E4M3FN)
    for (int e = 0; e < E; ++e)
      if (int rc = hdmoe_check_scale_in13("hdmoe_grouped_swiglu", experts[e], e)) return rc;
  if (rows_total == 0) return HDMOE_OK;
  return hdmoe_launch_ffn_gemm(true, weight_dtype, static_cast<const uint8_t*>(a), offsets, rows_total, E, experts,
                               static_cast<uint8_t*>(h), nullptr, 0, nullptr, nullptr, D, H, 0, 0,
                               static_cast<hipStream_t>(stream), "hdmoe_grouped_swiglu");
}

extern "C" int hdmoe_grouped_down(int weight_dtype, const void* h, const int32_t* offsets, int rows_total, int E, int H,
                                  int D, const hdmoe_ffn_weights* experts, void* y_bf16, hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(h);
  HDMOE_REQUIRE_PTR(offsets);
  HDMOE_REQUIRE_PTR(experts);
  HDMOE_REQUIRE_PTR(y_bf16);
  if (E < 1 || E > HDMOE_MAX_EXPERTS) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_grouped_down: E=%d", E);
  if (int rc = hdmoe_check_gemm_shape("hdmoe_grouped_down", weight_dtype, rows_total, H, D, BN)) return rc;
  if (rows_total == 0) return HDMOE_OK;
  return hdmoe_launch_ffn_gemm(false, weight_dtype, static_cast<const uint8_t*>(h), offsets, rows_total, E, experts,
                               static_cast<uint8_t*>(y_bf16), nullptr, 0, nullptr, nullptr, H, D, 0, 0,
                               static_cast<hipStream_t>(stream), "hdmoe_grouped_down");
}

extern "C" int hdmoe_linear(int weight_dtype, const void* a, int rows, int K, int N, const void* w,
                            const float* scale_w_dev, const float* scale_in_dev, void* out_bf16,
                            hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(a);
  HDMOE_REQUIRE_PTR(w);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (int rc = hdmoe_check_gemm_shape("hdmoe_linear", weight_dtype, rows, K, N, BN)) return rc;
  if (weight_dtype == HDMOE_W_E4M3FN) HDMOE_REQUIRE_PTR(scale_w_dev);
  if (rows == 0) return HDMOE_OK;
  hdmoe_ffn_weights fw;
  memset(&fw, 0, sizeof(fw));
  fw.w2 = w;
  fw.scale_w2 = scale_w_dev;
  fw.scale_in2 = scale_in_dev;
  return hdmoe_launch_ffn_gemm(false, weight_dtype, nullptr, nullptr, 0, 0, nullptr, nullptr,
                               static_cast<const uint8_t*>(a), rows, &fw, static_cast<uint8_t*>(out_bf16), 0, 0, K, N,
                               static_cast<hipStream_t>(stream), "hdmoe_linear");
}

extern "C" int hdmoe_linear_bias(int weight_dtype, const void* a, int rows, int K, int N, const void* w,
                                 const float* scale_w_dev, const float* scale_in_dev, const void* bias_bf16,
                                 void* out_bf16, hdmoe_stream_t stream) {
  if (bias_bf16 == nullptr && weight_dtype != HDMOE_W_F16)
    return hdmoe_linear(weight_dtype, a, rows, K, N, w, scale_w_dev, scale_in_dev, out_bf16, stream);
  HDMOE_REQUIRE_PTR(a);
  HDMOE_REQUIRE_PTR(w);
  HDMOE_REQUIRE_PTR(out_bf16);
  if (int rc = hdmoe_check_gemm_shape("hdmoe_linear_bias", weight_dtype == HDMOE_W_F16 ? HDMOE_W_BF16 : weight_dtype,
                                      rows, K, N, BN))
    return rc;
  if (weight_dtype == HDMOE_W_E4M3FN) HDMOE_REQUIRE_PTR(scale_w_dev);
  if (rows == 0) return HDMOE_OK;
  return hdmoe_launch_linear_bias(weight_dtype, static_cast<const uint8_t*>(a), rows, K, N,
                                  static_cast<const uint8_t*>(w), scale_w_dev, scale_in_dev,
                                  static_cast<const uint16_t*>(bias_bf16), static_cast<uint8_t*>(out_bf16),
                                  static_cast<hipStream_t>(stream), "hdmoe_linear_bias");
}

namespace {
int grouped_linear_entry(const char* what, bool f16, const void* a_bf16, const int32_t* offsets, int rows_total, int E,
                         const hdmoe_linear_weights* experts, void* out_bf16, const void* a_static_bf16,
                         int rows_static, const hdmoe_linear_weights* shared, void* out_static_bf16, int K, int N, int act,
                         hdmoe_stream_t stream, const int32_t* perm = nullptr, int T = 0) {
  if (perm != nullptr && (T <= 0 || rows_total != T * HDMOE_TOPK))
    return hdmoe_fail(HDMOE_E_SHAPE, "%s: rows_total=%d is not %d slots of T=%d tokens", what, rows_total, HDMOE_TOPK, T);
  if (E < 0 || E > HDMOE_MAX_EXPERTS) return hdmoe_fail(HDMOE_E_SHAPE, "%s: E=%d", what, E);
  if (act != HDMOE_ACT_NONE && act != HDMOE_ACT_GELU) return hdmoe_fail(HDMOE_E_SHAPE, "%s: act=%d", what, act);
  if (E > 0) {
    HDMOE_REQUIRE_PTR(a_bf16);
    HDMOE_REQUIRE_PTR(offsets);
    HDMOE_REQUIRE_PTR(experts);
    HDMOE_REQUIRE_PTR(out_bf16);
  }
  if (rows_static > 0) {
    HDMOE_REQUIRE_PTR(a_static_bf16);
    HDMOE_REQUIRE_PTR(shared);
    HDMOE_REQUIRE_PTR(out_static_bf16);
  }
  if (rows_static < 0) return hdmoe_fail(HDMOE_E_SHAPE, "%s: rows_static=%d", what, rows_static);
  const long rows_max = rows_total > rows_static ? rows_total : rows_static;
  if (int rc = hdmoe_check_gemm_shape(what, HDMOE_W_BF16, rows_max, K, N, BN)) return rc;  // same sizes for fp16
  if ((E == 0 || rows_total == 0) && rows_static == 0) return HDMOE_OK;
  return hdmoe_launch_linear_groups(static_cast<const uint8_t*>(a_bf16), offsets, rows_total, rows_total > 0 ? E : 0,
                                    experts, static_cast<uint8_t*>(out_bf16), static_cast<const uint8_t*>(a_static_bf16),
                                    rows_static, shared, static_cast<uint8_t*>(out_static_bf16), K, N, act,
                                    static_cast<hipStream_t>(stream), what, f16, perm, T, perm != nullptr ? 1 : 0);
}
}  // namespace

extern "C" int hdmoe_grouped_linear(const void* a_bf16, const int32_t* offsets, int rows_total, int E,
                                    const hdmoe_linear_weights* experts, void* out_bf16, const void* a_static_bf16,
                                    int rows_static, const hdmoe_linear_weights* shared, void* out_static_bf16, int K,
                                    int N, int act, hdmoe_stream_t stream) {
  return grouped_linear_entry("hdmoe_grouped_linear", false, a_bf16, offsets, rows_total, E, experts, out_bf16,
                              a_static_bf16, rows_static, shared, out_static_bf16, K, N, act, stream);
}

extern "C" int hdmoe_grouped_linear_f16(const void* a_f16, const int32_t* offsets, int rows_total, int E,
                                        const hdmoe_linear_weights* experts, void* out_f16, const void* a_static_f16,
                                        int rows_static, const hdmoe_linear_weights* shared, void* out_static_f16,
                                        int K, int N, int act, hdmoe_stream_t stream) {
  return grouped_linear_entry("hdmoe_grouped_linear_f16", true, a_f16, offsets, rows_total, E, experts, out_f16,
                              a_static_f16, rows_static, shared, out_static_f16, K, N, act, stream);
}

// The first Linear of the experts on the tokens themselves: sorted row r is token perm[r] / 2 (the rows the boolean
// masks of the reference select, read through the dispatch permutation instead of from a copy in expert order).
extern "C" int hdmoe_grouped_linear_tokens(int act_dtype, const void* x, int T, const int32_t* perm,
                                           const int32_t* offsets, int E, const hdmoe_linear_weights* experts, void* out,
                                           const hdmoe_linear_weights* shared, void* out_shared, int K, int N, int act,
                                           hdmoe_stream_t stream) {
  HDMOE_REQUIRE_PTR(perm);
  if (act_dtype != HDMOE_W_BF16 && act_dtype != HDMOE_W_F16)
    return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_grouped_linear_tokens: act_dtype=%d is neither HDMOE_W_BF16 nor HDMOE_W_F16",
                      act_dtype);
  if (T < 0 || E < 1) return hdmoe_fail(HDMOE_E_SHAPE, "hdmoe_grouped_linear_tokens: T=%d E=%d", T, E);
  if (T == 0) return HDMOE_OK;
  return grouped_linear_entry("hdmoe_grouped_linear_tokens", act_dtype == HDMOE_W_F16, x, offsets, T * HDMOE_TOPK, E,
                              experts, out, x, shared != nullptr ? T : 0, shared, out_shared, K, N, act, stream, perm, T);
}
