"""ctypes binding of libhdmoe.so (the C ABI declared in include/hdmoe.h).

The library is the only compute path of this package: if it is missing the import
of this module raises, there is no fallback.
"""
import ctypes
import os

# torch must be imported before the library is loaded: libhdmoe.so depends on libamdhip64 by soname,
# and the process must end up with the ONE HIP runtime torch brings, not a second copy.
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhdmoe.so")

W_BF16 = 0
W_E4M3FN = 1
W_F16 = 2
SRC_BF16 = 0
SRC_F32 = 2
ACT_NONE = 0
ACT_GELU = 1
MAX_EXPERTS = 16
E_NULL, E_SHAPE, E_WORKSPACE, E_LAUNCH = -1, -2, -3, -4
TOPK = 2
NUM_STAGES = 6
FORM_SWIGLU4W, FORM_LIGHT = 0, 1
FORM_AUTO, FORM_NEVER, FORM_ALWAYS = -1, 0, 1
STAGE_NAMES = ("gate", "dispatch", "quant_permute", "gemm_gate_up", "gemm_down", "combine")

c_void_p = ctypes.c_void_p
c_int = ctypes.c_int
c_int64 = ctypes.c_int64
c_size_t = ctypes.c_size_t


class FfnWeights(ctypes.Structure):
    """hdmoe_ffn_weights"""
    _fields_ = [
        ("w1", c_void_p), ("w2", c_void_p), ("w3", c_void_p),
        ("scale_w1", c_void_p), ("scale_w2", c_void_p), ("scale_w3", c_void_p),
        ("scale_in1", c_void_p), ("scale_in2", c_void_p), ("scale_in3", c_void_p),
        ("same_scale_in13", c_int),
    ]


class LinearWeights(ctypes.Structure):
    """hdmoe_linear_weights"""
    _fields_ = [("weight", c_void_p), ("bias", c_void_p)]


class LayerArgs(ctypes.Structure):
    """hdmoe_layer_args"""
    _fields_ = [
        ("T", c_int), ("D", c_int), ("H", c_int), ("Hs", c_int), ("E", c_int), ("weight_dtype", c_int),
        ("x", c_void_p), ("gate_w", c_void_p),
        ("experts", ctypes.POINTER(FfnWeights)), ("shared", ctypes.POINTER(FfnWeights)),
        ("out", c_void_p), ("workspace", c_void_p), ("workspace_bytes", c_size_t),
        ("topk_idx", c_void_p), ("topk_weight", c_void_p),
        ("stage_events", ctypes.POINTER(c_void_p)),
        ("mod_scale", c_void_p), ("mod_shift", c_void_p), ("mod_gate", c_void_p),
        ("tokens_per_batch", c_int), ("ln_eps", ctypes.c_float), ("uniform_scale_in", c_int),
        ("scale_check", c_void_p), ("fixed_k_cut", c_int),
    ]


class LayerLayout(ctypes.Structure):
    """hdmoe_layer_layout"""
    _fields_ = [(n, c_size_t) for n in
                ("topk_idx", "topk_weight", "counts", "offsets", "perm", "inv_perm", "dispatch_ws",
                 "a", "h", "y", "normed", "partials", "flags", "total")]


# name -> (restype, argtypes); every symbol include/hdmoe.h declares
SIGNATURES = {
    "hdmoe_version": (c_int, []),
    "hdmoe_last_error": (ctypes.c_char_p, []),
    "hdmoe_set_kernel_form": (c_int, [c_int, c_int]),
    "hdmoe_get_kernel_form": (c_int, [c_int]),
    "hdmoe_gate_up_kernel_name": (ctypes.c_char_p, [c_int, c_int, c_int, c_int, c_int, c_int, c_int]),
    "hdmoe_gate_top2": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "hdmoe_gate_top2_f16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "hdmoe_renorm_top2_bf16": (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    "hdmoe_dispatch_workspace_bytes": (c_size_t, [c_int, c_int]),
    "hdmoe_dispatch": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_size_t,
                               c_void_p]),
    "hdmoe_dispatch_static_max_tokens": (c_int, [c_int]),
    "hdmoe_dispatch_static": (c_int, [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "hdmoe_quant_fp8": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p]),
    "hdmoe_quant_permute_fp8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                        ctypes.POINTER(c_void_p), c_void_p, c_void_p]),
    "hdmoe_permute_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "hdmoe_grouped_swiglu": (c_int, [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                     ctypes.POINTER(FfnWeights), c_void_p, c_void_p]),
    "hdmoe_grouped_down": (c_int, [c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                   ctypes.POINTER(FfnWeights), c_void_p, c_void_p]),
    "hdmoe_linear": (c_int, [c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "hdmoe_linear_bias": (c_int, [c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_void_p]),
    "hdmoe_silu_mul_bf16": (c_int, [c_void_p, c_void_p, c_int64, c_void_p, c_void_p]),
    "hdmoe_gelu_bf16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "hdmoe_gelu_f16": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "hdmoe_scale_to_bf16": (c_int, [c_int, c_void_p, c_int64, c_void_p, c_void_p, c_void_p]),
    "hdmoe_grouped_linear": (c_int, [c_void_p, c_void_p, c_int, c_int, ctypes.POINTER(LinearWeights), c_void_p, c_void_p,
                                     c_int, ctypes.POINTER(LinearWeights), c_void_p, c_int, c_int, c_int, c_void_p]),
    "hdmoe_grouped_linear_f16": (c_int, [c_void_p, c_void_p, c_int, c_int, ctypes.POINTER(LinearWeights), c_void_p,
                                         c_void_p, c_int, ctypes.POINTER(LinearWeights), c_void_p, c_int, c_int, c_int,
                                         c_void_p]),
    "hdmoe_grouped_linear_tokens": (c_int, [c_int, c_void_p, c_int, c_void_p, c_void_p, c_int, ctypes.POINTER(LinearWeights),
                                            c_void_p, ctypes.POINTER(LinearWeights), c_void_p, c_int, c_int, c_int,
                                            c_void_p]),
    "hdmoe_stochastic_round_e4m3fn": (c_int, [c_int, c_void_p, ctypes.c_int64, c_void_p, ctypes.c_uint64, c_void_p,
                                              c_void_p]),
    "hdmoe_ln_modulate_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, ctypes.c_float, c_void_p,
                                       c_void_p]),
    "hdmoe_combine_gated_residual": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                             c_int, c_void_p, c_void_p]),
    "hdmoe_gated_residual_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "hdmoe_combine": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "hdmoe_combine_f16": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "hdmoe_layer_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "hdmoe_moe_ffn": (c_int, [ctypes.POINTER(LayerArgs), c_void_p]),
    "hdmoe_ffn_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "hdmoe_ffn_swiglu": (c_int, [c_int, c_void_p, c_int, c_int, c_int, ctypes.POINTER(FfnWeights), c_void_p, c_void_p,
                                 c_size_t, c_void_p]),
    "hdmoe_layer_layout_get": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, ctypes.POINTER(LayerLayout)]),
}


class HdmoeError(RuntimeError):
    def __init__(self, code, message):
        super().__init__(f"libhdmoe error {code}: {message}")
        self.code = code


def _load():
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing. Build it with `python -m comfyui_amd.build` (needs hipcc); "
            "comfyui_amd has no other compute path.")
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    return lib


lib = _load()


def check(rc):
    """Raise HdmoeError for a negative return code of an entry point."""
    if rc != 0:
        raise HdmoeError(rc, lib.hdmoe_last_error().decode("utf-8", "replace"))


def set_kernel_form(which, value):
    """hdmoe_set_kernel_form: FORM_SWIGLU4W / FORM_LIGHT to FORM_AUTO / FORM_NEVER / FORM_ALWAYS."""
    check(lib.hdmoe_set_kernel_form(which, value))


def ptr(t):
    """Device (or host) address of a tensor, None -> NULL."""
    return None if t is None else t.data_ptr()
