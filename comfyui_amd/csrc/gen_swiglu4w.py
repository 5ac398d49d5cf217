#!/usr/bin/env python3
"""Writes swiglu4w_asm.inc: the assembly bodies of the 4-wave fp8 gate/up kernel (swiglu4w.h).

    python comfyui_amd/csrc/gen_swiglu4w.py            # rewrites comfyui_amd/csrc/swiglu4w_asm.inc
    python comfyui_amd/csrc/gen_swiglu4w.py --check    # exit 1 if the file on disk differs

The kernel runs one wave per SIMD (4 waves, 512 registers each) on a 256-token x 256-weight-row tile and keeps
the SiLU*mul epilogue of a tile off the critical path: when a tile's K loop ends its accumulators are scaled,
rounded to bf16 and packed two to a register ("phase 1"), and the rest of the epilogue ("phase 2": SiLU, product,
rounding points, e4m3 cast, transpose through LDS, stores) is issued a few instructions at a time between the MFMAs
of the next tile's K loop. That needs a fixed register map and a schedule written instruction by instruction, which
is what this script produces; the order of LDS requests is simulated here so that every MFMA waits for exactly the
fragment reads it needs (LDS returns in order, lgkmcnt counts requests not yet returned).

Register map (per wave):
  a[0:255]    accumulators acc[ft][tt] = a[(4*ft + tt)*16 : +15]; ft 0,1 = w1 rows, ft 2,3 = the same features of w3
  v[128:255]  deferred outputs D[c][i] = v[128 + 16*c + i], c = 2*tt + f2 (the order phase 2 takes them in):
              bf16(w1 x) in the low half, bf16(w3 x) in the high half. Phase 2 always works on block 0 and then moves
              the other blocks down by one, so one body serves every block
  v[64:95]    weight fragments fb[ft] = v[64 + 8*ft : +7]
  v[96:127]   token fragments  fa[tt] = v[96 + 8*tt : +7]
  v[32:63]    addresses and temporaries (CTX below)
  v[0:31]     left to the compiler
"""
import os
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
OUT = os.path.join(HERE, "swiglu4w_asm.inc")

# ---- context registers v[32:63] -------------------------------------------------------------------------------
TOK_ADDR = {(0, 0): 32, (0, 1): 33, (1, 0): 34, (1, 1): 35}   # [K slice][16-byte half] LDS address of token reads
W_ADDR = {(0, 0): 36, (0, 1): 37, (1, 0): 38, (1, 1): 39}     # same for weight reads (includes the weight tile offset)
TOK_VOFF = [40 + j for j in range(8)]                         # global byte offset of the lane's row of token slab j
W_VOFF = 48                                                   # same for the weight rows (slab offset goes in an SGPR)
STG_WR = [49, 50]                                             # staging write address of feature quads q>>1 = 0, 1 (xor 32 flips f2)
STG_RD = 53                                                   # staging read address of the lane
OUT_VOFF = 54                                                 # output byte offset of the lane inside a 32-token block
TMP_P = 55
TMP = [56, 57, 58, 59, 60, 61, 62, 63]                        # phase 2 temporaries / store data (even-aligned tuples)

A_STAGE = 32768          # bytes of one stage of the token tile (256 rows x 128) = of the weight tile
FT_OFF = [0, 4096, 16384, 20480]   # weight fragment ft inside a stage of the weight tile
TT_OFF = [0, 4096, 8192, 12288]    # token fragment tt inside a stage of the token tile
W_TILE = 65536           # LDS offset of the weight stages ([A0|A1|B0|B1])
STG_OFF = 131072         # staging: 2 KiB per wave

# scratch SGPRs named in the clobber list of every statement
S_T0, S_T1, S_T2 = "s94", "s95", "s96"


def fb(ft):
    return f"v[{64 + 8 * ft}:{71 + 8 * ft}]"


def fa(tt):
    return f"v[{96 + 8 * tt}:{103 + 8 * tt}]"


def acc(ft, tt):
    b = (4 * ft + tt) * 16
    return f"a[{b}:{b + 15}]"


def dreg(c, i):
    return 128 + 16 * c + i


# MFMA order of a slice: row pairs (0,1) then (2,3), token blocks inside. Every fragment is refilled right after
# its last use and first used again 7 or more MFMAs later.
ORDER = [(ft, tt) for pair in ((0, 1), (2, 3)) for tt in range(4) for ft in pair]
REFILL_AFTER = {6: ["fb0"], 7: ["fb1"], 9: ["fa0"], 11: ["fa1"], 13: ["fa2"], 14: ["fb2"], 15: ["fa3", "fb3"]}


class Emitter:
    def __init__(self):
        self.lines = []
        self.lgkm = []          # tags of LDS requests issued and not known to have returned, oldest first

    def emit(self, s):
        self.lines.append(s)

    def lds(self, s, tag):
        self.lines.append(s)
        self.lgkm.append(tag)

    def wait_lgkm(self, tags):
        """Wait until every outstanding request carrying one of `tags` has returned."""
        last = -1
        for i, t in enumerate(self.lgkm):
            if t in tags:
                last = i
        if last < 0:
            return
        after = len(self.lgkm) - 1 - last
        n = min(after, 15)
        self.lines.append(f"s_waitcnt lgkmcnt({n})")
        # everything up to the (len - n)th request has returned
        self.lgkm = self.lgkm[len(self.lgkm) - n:] if n > 0 else []

    def wait_all(self, vm=True):
        self.lines.append("s_waitcnt vmcnt(0) lgkmcnt(0)" if vm else "s_waitcnt lgkmcnt(0)")
        self.lgkm = []


def frag_read(e, name, stage, ks):
    """Two ds_read_b128 of fragment `name` (fb0..3 / fa0..3) from slice ks of `stage`."""
    kind, idx = name[:2], int(name[2])
    if kind == "fb":
        reg, addr, off = 64 + 8 * idx, W_ADDR, stage * A_STAGE + FT_OFF[idx]
    else:
        reg, addr, off = 96 + 8 * idx, TOK_ADDR, stage * A_STAGE + TT_OFF[idx]
    e.lds(f"ds_read_b128 v[{reg}:{reg + 3}], v{addr[(ks, 0)]} offset:{off}", name)
    e.lds(f"ds_read_b128 v[{reg + 4}:{reg + 7}], v{addr[(ks, 1)]} offset:{off}", name)


def global_loads(stage, so):
    """The wave's 16 global->LDS loads of one K step into `stage` (K byte offset in SGPR operand `so`), as a list
    of instruction groups (one load each)."""
    groups = []
    for j in range(8):   # token slabs
        groups.append([f"s_add_u32 m0, %[ldsw], {stage * A_STAGE + j * 4096}", "s_nop 0",
                       f"buffer_load_dwordx4 v{TOK_VOFF[j]}, %[ra], %[{so}] offen lds"])
    for j in range(8):   # weight slabs: 0-3 from w1, 4-7 from w3
        rs = "rb0" if j < 4 else "rb1"
        g = []
        if j & 3:
            g.append(f"s_mul_i32 {S_T0}, %[kb32], {j & 3}")
            g.append(f"s_add_u32 {S_T0}, {S_T0}, %[{so}]")
            soff = S_T0
        else:
            soff = f"%[{so}]"
        g += [f"s_add_u32 m0, %[ldsw], {W_TILE + stage * A_STAGE + j * 4096}", "s_nop 0",
              f"buffer_load_dwordx4 v{W_VOFF}, %[{rs}], {soff} offen lds"]
        groups.append(g)
    return groups


def phase2_chunk():
    """Phase 2 of the 16 outputs of deferred block 0: list of (instruction, kind, cycles) with kind in {"v", "lds_w"}.
    Per output: g = low half, u = high half (bf16 as fp32); s = bf16(g / (1 + exp(-g))); m = bf16(s * u);
    o = e4m3fn(bf16(bf16(m) * inv_next)). A lane holds 4 consecutive features of one token per quad q. Afterwards
    the staging addresses flip to the other 32-feature half and blocks 1..7 move down by one."""
    ops = []
    t = TMP
    for q in range(4):
        for half in range(2):
            da, db = dreg(0, q * 4 + half * 2), dreg(0, q * 4 + half * 2 + 1)
            ga, ua, gb, ub, ta, tb = t[0], t[1], t[2], t[3], t[4], t[5]
            ops += [
                (f"v_lshlrev_b32 v{ga}, 16, v{da}", "v", 4), (f"v_and_b32 v{ua}, 0xffff0000, v{da}", "v", 4),
                (f"v_lshlrev_b32 v{gb}, 16, v{db}", "v", 4), (f"v_and_b32 v{ub}, 0xffff0000, v{db}", "v", 4),
                (f"v_mul_f32 v{ta}, 0xbfb8aa3b, v{ga}", "v", 4), (f"v_mul_f32 v{tb}, 0xbfb8aa3b, v{gb}", "v", 4),
                (f"v_exp_f32 v{ta}, v{ta}", "v", 16), (f"v_exp_f32 v{tb}, v{tb}", "v", 16),
                (f"v_add_f32 v{ta}, 1.0, v{ta}", "v", 4), (f"v_add_f32 v{tb}, 1.0, v{tb}", "v", 4),
                (f"v_rcp_f32 v{ta}, v{ta}", "v", 16), (f"v_rcp_f32 v{tb}, v{tb}", "v", 16),
                (f"v_mul_f32 v{ta}, v{ga}, v{ta}", "v", 4), (f"v_mul_f32 v{tb}, v{gb}, v{tb}", "v", 4),
                (f"v_cvt_pk_bf16_f32 v{TMP_P}, v{ta}, v{tb}", "v", 4),
                (f"v_lshlrev_b32 v{ta}, 16, v{TMP_P}", "v", 4), (f"v_and_b32 v{tb}, 0xffff0000, v{TMP_P}", "v", 4),
                (f"v_mul_f32 v{ta}, v{ta}, v{ua}", "v", 4), (f"v_mul_f32 v{tb}, v{tb}, v{ub}", "v", 4),
                (f"v_cvt_pk_bf16_f32 v{TMP_P}, v{ta}, v{tb}", "v", 4),
                (f"v_lshlrev_b32 v{ta}, 16, v{TMP_P}", "v", 4), (f"v_and_b32 v{tb}, 0xffff0000, v{TMP_P}", "v", 4),
                (f"v_mul_f32 v{ta}, %[inv], v{ta}", "v", 4), (f"v_mul_f32 v{tb}, %[inv], v{tb}", "v", 4),
                (f"v_cvt_pk_bf16_f32 v{TMP_P}, v{ta}, v{tb}", "v", 4),
                (f"v_cvt_scalef32_pk_fp8_bf16 v{t[6]}, v{TMP_P}, 1.0" + (" op_sel:[0,0,1]" if half else ""), "v", 4),
            ]
        # 4 bytes: features f2*32 + q*8 + hi*4 .. +3 of the lane's token
        ops.append((f"ds_write_b32 v{STG_WR[q >> 1]}, v{t[6]} offset:{(q & 1) * 8}", "lds_w", 4))
    for r in STG_WR:
        ops.append((f"v_xor_b32 v{r}, 32, v{r}", "v", 4))
    for c in range(7):
        for i in range(16):
            ops.append((f"v_mov_b32 v{dreg(c, i)}, v{dreg(c + 1, i)}", "v", 4))
    return ops


def read_back(e):
    """Token block back from the staging rows: 16 bytes per lane, two passes of 16 rows."""
    e.lds(f"ds_read_b128 v[{TMP[0]}:{TMP[3]}], v{STG_RD}", "stg")
    e.lds(f"ds_read_b128 v[{TMP[4]}:{TMP[7]}], v{STG_RD} offset:1024", "stg")


def emit_stores(e, soff):
    """The two 16-row passes of a token block; soff: SGPR (or operand) holding the block's first row offset. The row
    offset goes into the vector offset: it is the only part of the address that the buffer's range check sees, and
    rows past the end of a partial tile must be dropped by it."""
    e.emit(f"v_add_u32 v{TMP_P}, {soff}, v{OUT_VOFF}")
    e.emit(f"buffer_store_dwordx4 v[{TMP[0]}:{TMP[3]}], v{TMP_P}, %[ro], 0 offen")
    e.emit(f"v_add_u32 v{TMP_P}, %[ldo16], v{TMP_P}")
    e.emit(f"buffer_store_dwordx4 v[{TMP[4]}:{TMP[7]}], v{TMP_P}, %[ro], 0 offen")


def mfma(ft, tt, zero_c):
    c = "0" if zero_c else acc(ft, tt)
    return f"v_mfma_f32_32x32x64_f8f6f4 {acc(ft, tt)}, {fb(ft)}, {fa(tt)}, {c}"


CANON = [n for name in ("fb0", "fb1", "fa0", "fa1", "fa2", "fb2", "fa3", "fb3") for n in (name, name)]
SLOT_BUDGET = 44     # cycles of phase 2 work behind one MFMA (a 16-pass MFMA keeps the matrix pipe busy for 64)


def pair_body(first, chunk, label):
    """One pair of K steps: step A out of stage 0, step B out of stage 1. Entry state: the 8 fragments of slice 0
    of stage 0 requested in the order fb0 fb1 fa0 fa1 fa2 fb2 fa3 fb3 (two requests each), nothing else in flight
    on the LDS counter. Exit state: the same for the next pair. chunk: phase 2 of deferred block 0 rides along;
    if operand odd is set the block completes a 32-token x 64-feature piece, which is then stored."""
    e = Emitter()
    e.lgkm = list(CANON)
    p2 = phase2_chunk() if chunk else []
    # slots that take phase 2 work: every MFMA of slices 0 and 2, MFMAs 0..5 of slices 1 and 3
    slots = [(s, p) for s in range(4) for p in range(16) if s in (0, 2) or p < 6]
    budget = SLOT_BUDGET
    assert sum(c for _, _, c in p2) <= budget * len(slots), sum(c for _, _, c in p2)
    pos = 0
    # (slice, refill source stage, refill K slice, barrier slice?)
    plan = [(0, 0, 1, False), (1, 1, 0, True), (2, 1, 1, False), (3, 0, 0, True)]
    for s, rstage, rks, barrier in plan:
        loads = global_loads(0 if s == 1 else 1, "so0" if s == 1 else "so1") if barrier else []
        for p, (ft, tt) in enumerate(ORDER):
            e.wait_lgkm({f"fb{ft}", f"fa{tt}"})
            e.emit(mfma(ft, tt, first and s == 0))
            if (s, p) in slots:
                spent = 0
                last_slot = (s, p) == slots[-1]
                while pos < len(p2) and (last_slot or spent + p2[pos][2] <= budget):
                    ins, kind, cyc = p2[pos]
                    if kind == "lds_w":
                        e.lds(ins, "stg")
                    else:
                        e.emit(ins)
                    spent += cyc
                    pos += 1
            if barrier and p == 6:
                if chunk and s == 3:
                    assert pos == len(p2)
                    # a completed piece is read back in front of the barrier and stored behind it
                    e.emit("s_cmp_lg_u32 %[odd], 0")
                    e.emit(f"s_cbranch_scc0 {label}1f")
                    read_back(e)
                    e.emit(f"{label}1:")
                # everyone's loads of the stage about to be read have landed; everyone is done reading the other
                e.wait_all()
                e.emit("s_barrier")
                if chunk and s == 3:
                    e.emit("s_cmp_lg_u32 %[odd], 0")
                    e.emit(f"s_cbranch_scc0 {label}2f")
                    emit_stores(e, "%[stt]")
                    e.emit(f"{label}2:")
            for name in REFILL_AFTER.get(p, []):
                frag_read(e, name, rstage, rks)
            if barrier and p >= 7 and loads:
                for g in loads[:2]:
                    for ins in g:
                        e.emit(ins)
                loads = loads[2:]
        assert not loads
    assert pos == len(p2)
    assert e.lgkm == CANON, e.lgkm
    return e.lines


def fill_body():
    e = Emitter()
    for name in ("fb0", "fb1", "fa0", "fa1", "fa2", "fb2", "fa3", "fb3"):
        frag_read(e, name, 0, 0)
    return e.lines


def phase1_body():
    """acc -> D: D[2*tt + f2][i] = pack(bf16(acc[f2][tt][i] * sg), bf16(acc[f2+2][tt][i] * su)). The wait states in
    front cover the distance between the last MFMA and the first read of an accumulator."""
    lines = ["s_nop 15", "s_nop 7"]
    for f2 in range(2):
        for tt in range(4):
            for i in range(16):
                g = (4 * f2 + tt) * 16 + i
                u = (4 * (f2 + 2) + tt) * 16 + i
                ta, tb = TMP[(2 * i) % 8], TMP[(2 * i + 1) % 8]
                lines += [f"v_accvgpr_read_b32 v{ta}, a{g}", f"v_accvgpr_read_b32 v{tb}, a{u}",
                          f"v_mul_f32 v{ta}, %[sg], v{ta}", f"v_mul_f32 v{tb}, %[su], v{tb}",
                          f"v_cvt_pk_bf16_f32 v{dreg(2 * tt + f2, i)}, v{ta}, v{tb}"]
    return lines


def drain_body():
    """Phase 2 of the last tile of a block, with nothing to hide it behind."""
    e = Emitter()
    for c in range(8):
        for ins, kind, _ in phase2_chunk():
            if kind == "lds_w":
                e.lds(ins, "stg")
            else:
                e.emit(ins)
        if c & 1:
            read_back(e)
            e.wait_all(vm=False)
            e.emit(f"s_mul_i32 {S_T2}, %[ldo16], {(c >> 1) * 2}")
            emit_stores(e, S_T2)
            # the stores read their data registers before the next block's math overwrites them
            e.emit("s_nop 7")
    e.emit("s_waitcnt vmcnt(0)")
    return e.lines


def generate():
    out = ["// Generated by gen_swiglu4w.py; do not edit. See that script for the register map and the schedule.", ""]
    # variants of the pair body, selected by operand var: bit 0 = phase 2 work rides along, bit 1 = first pair of a
    # tile (the accumulators start from zero)
    body = []
    for code in (1, 2, 3):
        body.append(f"s_cmp_eq_u32 %[var], {code}")
        body.append(f"s_cbranch_scc1 {10 + code}0f")
    for code in (0, 1, 2, 3):
        body.append(f"{10 + code}0:")
        body += pair_body(bool(code & 2), bool(code & 1), str(10 + code))
        if code != 3:
            body.append("s_branch 199f")
    body.append("199:")
    for name, lines in (("HDMOE4W_PAIR_ASM", body), ("HDMOE4W_FILL_ASM", fill_body()),
                        ("HDMOE4W_PHASE1_ASM", phase1_body()), ("HDMOE4W_DRAIN_ASM", drain_body())):
        out.append(f"#define {name} \\")
        out.append(" \\\n".join('  "' + ln + '\\n"' for ln in lines))
        out.append("")
    return "\n".join(out)


if __name__ == "__main__":
    text = generate()
    if "--check" in sys.argv:
        sys.exit(0 if os.path.exists(OUT) and open(OUT).read() == text else 1)
    with open(OUT, "w") as f:
        f.write(text)
    print("wrote", OUT, len(text.splitlines()), "lines")
