"""comfyui_amd/csrc/swiglu4w_asm.inc is generated; the file in the tree must be what the generator writes."""
import os
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_generated_assembly_is_up_to_date():
    gen = os.path.join(ROOT, "comfyui_amd", "csrc", "gen_swiglu4w.py")
    r = subprocess.run([sys.executable, gen, "--check"])
    assert r.returncode == 0, "run python comfyui_amd/csrc/gen_swiglu4w.py and rebuild"


def test_schedule_invariants():
    """Every pair body leaves the LDS request queue in the state the next one assumes, spreads no more phase 2
    work behind an MFMA than fits in its shadow, and contains 64 MFMAs (4 slices of 16)."""
    sys.path.insert(0, os.path.join(ROOT, "comfyui_amd", "csrc"))
    try:
        import gen_swiglu4w as G
    finally:
        sys.path.pop(0)
    for first in (False, True):
        for chunk in (False, True):
            lines = G.pair_body(first, chunk, "9")
            assert sum(ln.startswith("v_mfma") for ln in lines) == 64
            assert sum(ln.startswith("buffer_load_dwordx4") for ln in lines) == 32
            assert sum(ln == "s_barrier" for ln in lines) == 2
            zero_c = sum(ln.startswith("v_mfma") and ln.endswith(", 0") for ln in lines)
            assert zero_c == (16 if first else 0)
    # each accumulator block is written by exactly one (ft, tt) and phase 1 reads every accumulator once
    p1 = G.phase1_body()
    reads = [ln for ln in p1 if ln.startswith("v_accvgpr_read")]
    assert len(reads) == 256 and len({ln.split(", ")[1] for ln in reads}) == 256
    packs = [ln for ln in p1 if ln.startswith("v_cvt_pk_bf16_f32")]
    assert len({ln.split()[1] for ln in packs}) == 128
