// fp8 gate/up GEMM + SiLU*mul with the epilogue of a tile hidden behind the K loop of the next one.
//
// Included by gemm.hip inside its unnamed namespace (uses GemmArgs, GemmGroup, swz, make_rsrc, lds_ptr_t).
//
// Same contraction, rounding points and LDS tile format as grouped_gemm_kernel<FP8_SWIGLU, TT>
// (/root/reference/comfy/ldm/hidream/model.py:238 behind /root/reference/comfy/ops.py:314-358), other shape of the
// work: 4 waves of 64 (one per SIMD, up to 512 registers each), block tile 256 tokens x 256 weight rows (the same
// 128 features of w1 and w3), wave tile 128 tokens x 128 weight rows with its 256 accumulators in the AGPR half
// of the register file. When a tile's K loop ends, the wave scales its accumulators, rounds them to bf16 and packs
// w1 x / w3 x pairs into 128 VGPRs (phase 1); SiLU, the product, the remaining rounding points, the e4m3 cast,
// the transpose through LDS and the stores (phase 2) are issued between the MFMAs of the next tile's first 16 K
// steps, 16 outputs per pair of steps. K steps of consecutive tiles form one stream: the loads of a tile's first
// two steps are requested during the last two steps of the tile before, so the matrix pipe does not drain between
// tiles. The instruction schedule is generated (gen_swiglu4w.py -> swiglu4w_asm.inc) with every register fixed.
//
// Limits (the launcher falls back to grouped_gemm_kernel otherwise): K a multiple of 256 bytes and at least 2048,
// every group with a scale_input for the consuming Linear (no clamp form of the cast), operand buffers under 2 GiB.
#include "swiglu4w_asm.inc"

constexpr int W4_THREADS = 256;
constexpr int W4_BM = 256;                        // tokens per block tile
constexpr int W4_FEAT = 128;                      // features per block tile
constexpr int W4_STAGE = 32768;                   // one stage of the token tile = of the weight tile
constexpr int W4_W_TILE = 65536;                  // LDS: [tok 0 | tok 1 | w 0 | w 1 | staging]
constexpr int W4_STG = 131072;
constexpr int W4_SMEM = W4_STG + 4 * 2048;

typedef float v32f __attribute__((ext_vector_type(32)));
typedef int v32i __attribute__((ext_vector_type(32)));

// positions in the context registers v[32:63] (gen_swiglu4w.py)
enum { W4_TOK_ADDR = 0, W4_W_ADDR = 4, W4_TOK_VOFF = 8, W4_W_VOFF = 16, W4_STG_WR = 17, W4_STG_RD = 21, W4_OUT_VOFF = 22 };

#define W4_STATE                                                                                                     \
  "+{a[0:31]}"(c0), "+{a[32:63]}"(c1), "+{a[64:95]}"(c2), "+{a[96:127]}"(c3), "+{a[128:159]}"(c4),                   \
      "+{a[160:191]}"(c5), "+{a[192:223]}"(c6), "+{a[224:255]}"(c7), "+{v[128:159]}"(d0), "+{v[160:191]}"(d1),      \
      "+{v[192:223]}"(d2), "+{v[224:255]}"(d3), "+{v[64:95]}"(fbv), "+{v[96:127]}"(fav), "+{v[32:63]}"(ctx)
#define W4_STATE_OUT                                                                                                 \
  "={a[0:31]}"(c0), "={a[32:63]}"(c1), "={a[64:95]}"(c2), "={a[96:127]}"(c3), "={a[128:159]}"(c4),                   \
      "={a[160:191]}"(c5), "={a[192:223]}"(c6), "={a[224:255]}"(c7), "={v[128:159]}"(d0), "={v[160:191]}"(d1),      \
      "={v[192:223]}"(d2), "={v[224:255]}"(d3), "={v[64:95]}"(fbv), "={v[96:127]}"(fav)
#define W4_CLOBBER "memory", "scc", "s94", "s95", "s96"

__global__ __launch_bounds__(W4_THREADS) __attribute__((amdgpu_waves_per_eu(1, 1))) void swiglu4w_kernel(const GemmArgs args) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wq = wave & 1, wt = wave >> 1;
  auto sgpr = [](int v) { return __builtin_amdgcn_readfirstlane(v); };

  // ---- tile enumeration: as grouped_gemm_kernel with one tile list cut in eighths ---------------------------
  int off_lane = 0;
  if (args.offsets != nullptr && lane <= args.n_offsets) off_lane = args.offsets[lane];
  auto seg = [&](const GemmGroup& gg, int& rb, int& re) {
    if (gg.row_begin >= 0) { rb = gg.row_begin; re = gg.row_end; }
    else { rb = __builtin_amdgcn_readlane(off_lane, gg.dyn); re = __builtin_amdgcn_readlane(off_lane, gg.dyn + 1); }
  };
  int total = 0;
  for (int g = 0; g < args.G; ++g) {
    int rb, re;
    seg(args.g[g], rb, re);
    total += ((re - rb + W4_BM - 1) / W4_BM) * (args.g[g].n_out / W4_FEAT);
  }
  const int per_xcd = (total + HDMOE_NUM_XCD - 1) / HDMOE_NUM_XCD;
  const int xcd = blockIdx.x % HDMOE_NUM_XCD, slot = blockIdx.x / HDMOE_NUM_XCD;
  const int nslots = gridDim.x / HDMOE_NUM_XCD;
  struct Tile4 { int g, row0, rows_here, n0; };
  auto decode = [&](int i) -> Tile4 {
    Tile4 d = {-1, 0, 0, 0};
    const int in_xcd = slot + i * nslots;
    int L = xcd * per_xcd + in_xcd;
    if (in_xcd >= per_xcd || L >= total) return d;
    int g = 0, rb = 0, re = 0, mtiles = 0, ntiles = 0;
    for (; g < args.G; ++g) {
      seg(args.g[g], rb, re);
      mtiles = (re - rb + W4_BM - 1) / W4_BM;
      ntiles = args.g[g].n_out / W4_FEAT;
      if (L < mtiles * ntiles) break;
      L -= mtiles * ntiles;
    }
    if (g >= args.G) return d;
    const int nbands = max(1, (mtiles + GROUP_M / 2) / GROUP_M);
    const int band = min(L / (GROUP_M * ntiles), nbands - 1);
    const int first_m = band * GROUP_M;
    const int gm = band == nbands - 1 ? mtiles - first_m : GROUP_M;
    const int within = L - band * (GROUP_M * ntiles);
    d.g = g;
    d.row0 = rb + (first_m + within % gm) * W4_BM;
    d.rows_here = min(re - d.row0, W4_BM);
    d.n0 = (within / gm) * W4_FEAT;
    return d;
  };

  // the gathered token operand: as the groups describe it, or the alternative the flag selects (GemmArgs::alt)
  const bool use_alt = args.alt.flag != nullptr && sgpr(*args.alt.flag) == 0;
  auto token_base = [&](const GemmGroup& gg) { return (use_alt && gg.gather != nullptr) ? args.alt.a : gg.a; };
  auto gather_shift = [&](const GemmGroup& gg) { return use_alt ? args.alt.shift : gg.gather_shift; };

  Tile4 cur = decode(0);
  if (cur.g < 0) return;   // block-uniform: every wave of the block leaves together
  Tile4 nxt = decode(1);

  // ---- addressing ---------------------------------------------------------------------------------------------
  const uint32_t lds0 = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  const int ld_row = wave * 8 + (lane >> 3);                 // row within a 32-row slab
  const int ld_chunk = (lane & 7) ^ swz(ld_row);
  const int ldsw = sgpr((int)lds0 + wave * 1024);
  const int fr_row = lane & 31, fr_grp = lane >> 5, fr_swz = swz(fr_row);

  v32f c0, c1, c2, c3, c4, c5, c6, c7;
  v32i d0, d1, d2, d3, fbv, fav, ctx;
#pragma unroll
  for (int i = 0; i < 32; ++i) ctx[i] = 0;
#pragma unroll
  for (int ks = 0; ks < 2; ++ks)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int c = (((ks * 4 + fr_grp * 2) ^ fr_swz) * 16) ^ (h * 16);
      ctx[W4_TOK_ADDR + ks * 2 + h] = (int)lds0 + (wt * 128 + fr_row) * 128 + c;
      ctx[W4_W_ADDR + ks * 2 + h] = (int)lds0 + W4_W_TILE + (wq * 64 + fr_row) * 128 + c;
    }
  {
    const int tok32 = lane & 31, hi32 = lane >> 5;
    const int stg = (int)lds0 + W4_STG + wave * 2048;
#pragma unroll
    for (int qh = 0; qh < 2; ++qh)
      ctx[W4_STG_WR + qh] = stg + tok32 * 64 + (((tok32 >> 1) & 1) << 5) + ((qh ^ (tok32 & 1)) << 4) + hi32 * 4;
    const int row = lane >> 2, c = lane & 3;
    ctx[W4_STG_RD] = stg + row * 64 + ((c ^ (row & 3)) << 4);
  }

  auto raw_rsrc = [](const void* p, uint32_t bytes) -> v4i {
    const uint64_t a = reinterpret_cast<uint64_t>(p);
    v4i r;
    r.x = (int)(uint32_t)a; r.y = (int)(uint32_t)((a >> 32) & 0xffffu); r.z = (int)bytes; r.w = 0x00020000;
    return r;
  };
  auto srsrc = [&](const v4i& r) -> v4i {
    v4i o;
    o.x = sgpr(r.x); o.y = sgpr(r.y); o.z = sgpr(r.z); o.w = sgpr(r.w);
    return o;
  };
  // row indices of the 8 token slabs of a tile (row r of the tile -> row of the operand buffer), -1 past its end
  auto load_rows = [&](const Tile4& d, int (&gi)[8]) {
    const GemmGroup& gg = args.g[d.g];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int r = j * 32 + ld_row;
      int v = -1;
      if (r < d.rows_here) v = gg.gather != nullptr ? (gg.gather[d.row0 + r] >> gather_shift(gg)) : d.row0 + r;
      gi[j] = v;
    }
  };
  // the tile whose K steps are being requested
  v4i ra = {0, 0, 0, 0}, rb0 = ra, rb1 = ra;
  int kbytes = 0;
  auto set_load_tile = [&](const Tile4& d, const int (&gi)[8]) {
    if (d.g < 0) {   // no further tile: the requests still go out, against empty buffers (zeros)
      ra = raw_rsrc(nullptr, 0); rb0 = ra; rb1 = ra;
      return;
    }
    const GemmGroup& gg = args.g[d.g];
    kbytes = gg.kbytes;
    ra = raw_rsrc(token_base(gg), 0x7fffffffu);   // rows are valid by construction; rows past the tile get an offset of 2^31
    rb0 = raw_rsrc(gg.b0 + (size_t)d.n0 * kbytes, (uint32_t)W4_FEAT * (uint32_t)kbytes);
    rb1 = raw_rsrc(gg.b1 + (size_t)d.n0 * kbytes, (uint32_t)W4_FEAT * (uint32_t)kbytes);
#pragma unroll
    for (int j = 0; j < 8; ++j) ctx[W4_TOK_VOFF + j] = gi[j] >= 0 ? gi[j] * kbytes + ld_chunk * 16 : (int)0x80000000u;
    ctx[W4_W_VOFF] = ld_row * kbytes + ld_chunk * 16;
  };

  int gi_cur[8], gi_nxt[8];
  load_rows(cur, gi_cur);
  set_load_tile(cur, gi_cur);

  // ---- first two K steps of the block's first tile, as a burst ------------------------------------------------
  {
    const __amdgpu_buffer_rsrc_t pa = make_rsrc(token_base(args.g[cur.g]), 0x7fffffffu);
    const __amdgpu_buffer_rsrc_t pb0 = make_rsrc(args.g[cur.g].b0 + (size_t)cur.n0 * kbytes, (uint32_t)W4_FEAT * (uint32_t)kbytes);
    const __amdgpu_buffer_rsrc_t pb1 = make_rsrc(args.g[cur.g].b1 + (size_t)cur.n0 * kbytes, (uint32_t)W4_FEAT * (uint32_t)kbytes);
#pragma unroll
    for (int st = 0; st < 2; ++st) {
      uint8_t* const base = smem + st * W4_STAGE + wave * 1024;
#pragma unroll
      for (int j = 0; j < 8; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(pa, (lds_ptr_t)(base + j * 4096), 16, ctx[W4_TOK_VOFF + j], st * BK, 0, 0);
#pragma unroll
      for (int j = 0; j < 8; ++j)
        __builtin_amdgcn_raw_ptr_buffer_load_lds(j < 4 ? pb0 : pb1, (lds_ptr_t)(base + W4_W_TILE + j * 4096), 16,
                                                 ctx[W4_W_VOFF], st * BK + (j & 3) * 32 * kbytes, 0, 0);
    }
  }
  __builtin_amdgcn_s_waitcnt(0x0f70);  // vmcnt(0)
  __syncthreads();
  asm volatile(HDMOE4W_FILL_ASM : W4_STATE_OUT, "+{v[32:63]}"(ctx) : : "memory");

  // ---- the stream of K step pairs -----------------------------------------------------------------------------
  // deferred tile (phase 2 in flight): output buffer, row pitch, cast scale
  v4i ro = raw_rsrc(nullptr, 0);
  int ldo16 = 0, inv_bits = 0;
  bool have_def = false;
  // per-tensor scales come through the scalar cache: waiting for a vector load here would also wait for every
  // global->LDS request in flight (one in-order counter)
  typedef const __attribute__((address_space(4))) float* const_float_ptr;
  auto scalar_load = [](const float* p) -> float { return *(const_float_ptr)(uintptr_t)p; };
  for (int i = 0;; ++i) {
    const GemmGroup& gg = args.g[cur.g];
    const float s_in = gg.s_in ? scalar_load(gg.s_in) : 1.0f;
    const int sg_bits = sgpr(__float_as_int(s_in * scalar_load(gg.sb0)));
    const int su_bits = sgpr(__float_as_int((gg.s_in_b ? scalar_load(gg.s_in_b) : s_in) * scalar_load(gg.sb1)));
    const int inv_next_bits = sgpr(__float_as_int(hdmoe_dev_round_bf16(__fdiv_rn(1.0f, scalar_load(gg.s_next)))));
    const int pairs = sgpr(gg.kbytes / (2 * BK));
    const int kb32 = sgpr(32 * gg.kbytes);
    if (nxt.g >= 0) load_rows(nxt, gi_nxt);   // lands during the K loop
    for (int j = 0; j < pairs; ++j) {
      const bool last = j == pairs - 1;
      if (last) set_load_tile(nxt, gi_nxt);
      const int so0 = sgpr(last ? 0 : (2 * j + 2) * BK), so1 = sgpr(last ? BK : (2 * j + 3) * BK);
      const int var = sgpr((j == 0 ? 2 : 0) | ((have_def && j < 8) ? 1 : 0));
      const int odd = sgpr(j & 1), stt = sgpr((j >> 1) * 2 * ldo16);
      const int kb = sgpr(last && nxt.g >= 0 ? 32 * args.g[nxt.g].kbytes : kb32);
      asm volatile(HDMOE4W_PAIR_ASM
                   : W4_STATE
                   : [ra] "s"(srsrc(ra)), [rb0] "s"(srsrc(rb0)), [rb1] "s"(srsrc(rb1)), [ro] "s"(srsrc(ro)), [so0] "s"(sgpr(so0)),
                     [so1] "s"(sgpr(so1)), [kb32] "s"(sgpr(kb)), [ldsw] "s"(sgpr(ldsw)), [var] "s"(sgpr(var)),
                     [odd] "s"(sgpr(odd)), [stt] "s"(sgpr(stt)),
                     [inv] "s"(sgpr(inv_bits)), [ldo16] "s"(sgpr(ldo16))
                   : W4_CLOBBER);
    }
    // phase 1: this tile's accumulators become the deferred tile
    {
      asm volatile(HDMOE4W_PHASE1_ASM : W4_STATE : [sg] "s"(sgpr(sg_bits)), [su] "s"(sgpr(su_bits)) : W4_CLOBBER);
      const int ldo = gg.n_out;   // fp8 output: one byte per feature
      ro = raw_rsrc(gg.out + (size_t)cur.row0 * ldo + cur.n0, (uint32_t)cur.rows_here * (uint32_t)ldo);
      ldo16 = 16 * ldo;
      inv_bits = inv_next_bits;
      ctx[W4_OUT_VOFF] = (wt * 128 + (lane >> 2)) * ldo + wq * 64 + (lane & 3) * 16;
      have_def = true;
    }
    if (nxt.g < 0) break;
    cur = nxt;
    nxt = decode(i + 2);
  }
  // ---- phase 2 of the last tile ------------------------------------------------------------------------------
  asm volatile(HDMOE4W_DRAIN_ASM
               : W4_STATE
               : [ro] "s"(srsrc(ro)), [inv] "s"(sgpr(inv_bits)), [ldo16] "s"(sgpr(ldo16))
               : W4_CLOBBER);
}

// Whether the launch fits swiglu4w_kernel (see the limits above).
inline bool swiglu4w_fits(const GemmArgs& args, long long max_operand_bytes) {
  if (args.G <= 0 || args.nparts != 1) return false;
  const int kb = args.g[0].kbytes;
  if (kb % (2 * BK) != 0 || kb < 16 * BK) return false;
  for (int g = 0; g < args.G; ++g) {
    const GemmGroup& gg = args.g[g];
    if (gg.kbytes != kb || gg.s_next == nullptr || gg.n_out % W4_FEAT != 0) return false;
  }
  return max_operand_bytes < (1ll << 31);
}
