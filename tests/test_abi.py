"""The C ABI without a GPU: libhdmoe.so loads, exports every function include/hdmoe.h declares, and rejects bad
arguments with the documented codes before touching the device."""
import ctypes
import os
import re

import pytest
import torch  # noqa: F401  (load order: torch's HIP runtime first)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "hdmoe.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hdmoe_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound():
    from comfyui_amd import _lib
    names = declared_functions()
    assert len(names) >= 17
    for n in names:
        assert hasattr(_lib.lib, n), n
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert sorted(_lib.SIGNATURES) == names
    version = int(re.search(r"#define\s+HDMOE_VERSION\s+(\d+)", open(HEADER).read()).group(1))
    assert _lib.lib.hdmoe_version() == version >= 101


def test_header_constants_match_binding():
    from comfyui_amd import _lib
    text = open(HEADER).read()
    consts = dict(re.findall(r"#define\s+(HDMOE_[A-Z0-9_]+)\s+\(?(-?\d+)\)?", text))
    assert int(consts["HDMOE_W_BF16"]) == _lib.W_BF16 and int(consts["HDMOE_W_E4M3FN"]) == _lib.W_E4M3FN
    assert int(consts["HDMOE_MAX_EXPERTS"]) == _lib.MAX_EXPERTS and int(consts["HDMOE_TOPK"]) == _lib.TOPK
    assert int(consts["HDMOE_NUM_STAGES"]) == _lib.NUM_STAGES == len(_lib.STAGE_NAMES)
    assert (int(consts["HDMOE_E_NULL"]), int(consts["HDMOE_E_SHAPE"]), int(consts["HDMOE_E_WORKSPACE"]),
            int(consts["HDMOE_E_LAUNCH"])) == (_lib.E_NULL, _lib.E_SHAPE, _lib.E_WORKSPACE, _lib.E_LAUNCH)
    assert ctypes.sizeof(_lib.FfnWeights) == 10 * 8
    assert ctypes.sizeof(_lib.LayerLayout) == 14 * 8


def test_struct_layouts_match_what_a_c_compiler_sees(tmp_path):
    """sizeof/offsetof of every struct of the header as gcc lays them out == the ctypes mirrors."""
    import subprocess
    from comfyui_amd import _lib
    structs = {"hdmoe_ffn_weights": _lib.FfnWeights, "hdmoe_layer_args": _lib.LayerArgs,
               "hdmoe_layer_layout": _lib.LayerLayout}
    lines = []
    for cname, cls in structs.items():
        lines.append(f'printf("{cname} %zu\\n", sizeof({cname}));')
        for fname, _ in cls._fields_:
            lines.append(f'printf("{cname}.{fname} %zu\\n", offsetof({cname}, {fname}));')
    src = tmp_path / "layout.c"
    src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "hdmoe.h"\nint main(void) {\n'
                   + "\n".join(lines) + "\nreturn 0; }\n")
    exe = tmp_path / "layout"
    subprocess.check_call(["gcc", "-std=c11", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)])
    got = dict(l.split() for l in subprocess.check_output([str(exe)], text=True).splitlines())
    for cname, cls in structs.items():
        assert int(got[cname]) == ctypes.sizeof(cls), cname
        for fname, _ in cls._fields_:
            assert int(got[f"{cname}.{fname}"]) == getattr(cls, fname).offset, f"{cname}.{fname}"


def test_argument_errors_are_reported_without_a_device():
    from comfyui_amd import _lib
    L = _lib.lib
    buf = (ctypes.c_char * 4096)()
    p = ctypes.addressof(buf)
    assert L.hdmoe_gate_top2(None, p, 4, 2560, 4, p, p, None) == _lib.E_NULL
    assert b"x_bf16" in L.hdmoe_last_error()
    assert L.hdmoe_gate_top2(p, p, 4, 2561, 4, p, p, None) == _lib.E_SHAPE
    assert L.hdmoe_gate_top2(p, p, 4, 2560, 1, p, p, None) == _lib.E_SHAPE
    assert L.hdmoe_gate_top2(p, p, 4, 2560, 17, p, p, None) == _lib.E_SHAPE
    assert L.hdmoe_gate_top2(p, p, 0, 2560, 4, p, p, None) == 0                 # empty input: nothing to do
    assert L.hdmoe_dispatch(p, 8, 17, p, p, p, p, p, 4096, None) == _lib.E_SHAPE
    assert L.hdmoe_dispatch(p, 100000, 4, p, p, p, p, p, 16, None) == _lib.E_WORKSPACE
    assert L.hdmoe_quant_fp8(p, 4, 2563, None, p, None) == _lib.E_SHAPE
    assert L.hdmoe_combine(p, p, p, None, 4, 12, p, None) == _lib.E_SHAPE
    assert L.hdmoe_linear(_lib.W_E4M3FN, p, 4, 100, 256, p, p, None, p, None) == _lib.E_SHAPE   # K not /128
    assert L.hdmoe_linear(_lib.W_E4M3FN, p, 4, 128, 200, p, p, None, p, None) == _lib.E_SHAPE   # N not /256
    assert L.hdmoe_linear(_lib.W_E4M3FN, p, 4, 128, 256, p, None, None, p, None) == _lib.E_NULL  # fp8 needs scale_weight
    assert L.hdmoe_linear(7, p, 4, 128, 256, p, p, None, p, None) == _lib.E_SHAPE
    assert L.hdmoe_linear(_lib.W_BF16, p, 0, 64, 256, p, None, None, p, None) == 0
    assert L.hdmoe_silu_mul_bf16(p, p, 12, p, None) == _lib.E_SHAPE
    # the fp16 entry points and the fp16 weight code
    assert L.hdmoe_gate_top2_f16(None, p, 4, 2048, 8, p, p, None) == _lib.E_NULL
    assert b"x_f16" in L.hdmoe_last_error()
    assert L.hdmoe_gate_top2_f16(p, p, 4, 2049, 8, p, p, None) == _lib.E_SHAPE
    assert L.hdmoe_gate_top2_f16(p, p, 0, 2048, 8, p, p, None) == 0
    assert L.hdmoe_combine_f16(p, p, p, None, 4, 12, p, None) == _lib.E_SHAPE
    assert L.hdmoe_gelu_f16(p, 12, p, None) == _lib.E_SHAPE
    assert L.hdmoe_grouped_linear_f16(p, p, 8, 17, None, p, None, 0, None, None, 256, 256, 0, None) == _lib.E_SHAPE
    assert L.hdmoe_grouped_linear_f16(p, p, 8, 2, None, p, None, 0, None, None, 256, 256, 0, None) == _lib.E_NULL
    assert L.hdmoe_linear(_lib.W_F16, p, 4, 128, 256, p, None, None, p, None) == _lib.E_SHAPE    # fp16: hdmoe_linear_bias only
    assert L.hdmoe_linear_bias(_lib.W_F16, p, 4, 100, 256, p, None, None, None, p, None) == _lib.E_SHAPE
    assert L.hdmoe_linear_bias(_lib.W_F16, p, 0, 128, 256, p, None, None, None, p, None) == 0
    assert L.hdmoe_layer_workspace_bytes(16, 2560, 6912, 3584, 4, _lib.W_F16) == 0               # the layer takes bf16 / fp8
    assert L.hdmoe_moe_ffn(None, None) == _lib.E_NULL
    args = _lib.LayerArgs()
    args.T, args.D, args.H, args.Hs, args.E, args.weight_dtype = 16, 2560, 6912, 3584, 4, _lib.W_E4M3FN
    args.x = args.gate_w = args.out = args.workspace = p
    arr = (_lib.FfnWeights * 4)()
    args.experts = arr
    args.shared = ctypes.pointer(_lib.FfnWeights())
    args.workspace_bytes = 1024
    assert L.hdmoe_moe_ffn(ctypes.byref(args), None) == _lib.E_WORKSPACE
    assert b"workspace" in L.hdmoe_last_error()


def test_layer_layout_is_consistent():
    from comfyui_amd import _lib
    for (T, D, H, Hs, E, code) in [(8192, 2560, 6912, 3584, 4, 1), (1024, 2560, 6912, 3584, 4, 0), (1, 256, 768, 512, 4, 1),
                                   (0, 256, 768, 0, 2, 1)]:
        lay = _lib.LayerLayout()
        assert _lib.lib.hdmoe_layer_layout_get(T, D, H, Hs, E, code, ctypes.byref(lay)) == 0
        offs = [getattr(lay, n) for n, _ in _lib.LayerLayout._fields_]
        assert offs[:-1] == sorted(offs[:-1]) and all(o % 256 == 0 for o in offs)
        assert lay.total == _lib.lib.hdmoe_layer_workspace_bytes(T, D, H, Hs, E, code)
        eb = 1 if code == 1 else 2
        assert lay.h - lay.a >= ((2 * T + (T if Hs else 0)) * D if code == 1 else 0)   # bf16: no copy of the tokens
        assert lay.y - lay.h >= (2 * T * H + T * Hs) * eb
        assert lay.total - lay.y >= (2 * T + (T if Hs else 0)) * D * 2
    assert _lib.lib.hdmoe_layer_workspace_bytes(8, 256, 768, 512, 99, 1) == 0


def test_static_dispatch_rejects_sizes_beyond_its_buffer():
    from comfyui_amd import _lib
    L = _lib.lib
    for E in (1, 4, 16):
        limit = L.hdmoe_dispatch_static_max_tokens(E)
        assert limit >= 1 << 20
        assert L.hdmoe_dispatch_workspace_bytes(limit, E) <= 64 * 1024
    limit = L.hdmoe_dispatch_static_max_tokens(16)
    assert L.hdmoe_dispatch_workspace_bytes(limit + 2048, 16) > 64 * 1024
    # nothing is enqueued for a refused size, so the buffers may be tiny
    t = torch.zeros(64, dtype=torch.int32)
    p = t.data_ptr()
    rc = L.hdmoe_dispatch_static(p, limit + 2048, 16, p, p, p, p, None)
    assert rc == _lib.E_WORKSPACE
    assert b"at most" in L.hdmoe_last_error()
    assert L.hdmoe_dispatch_static(p, 8, 17, p, p, p, p, None) == _lib.E_SHAPE
    assert L.hdmoe_dispatch_static(None, 8, 4, p, p, p, p, None) == _lib.E_NULL
