"""Tensor-level wrappers over the C ABI: they check devices/dtypes/shapes, allocate
outputs with torch (device memory and stream plumbing only) and enqueue the HIP
kernels on torch's current stream. Nothing here computes with torch.
"""
import ctypes

import torch

from . import _lib
from ._lib import FfnWeights, LayerArgs, LayerLayout, LinearWeights, W_BF16, W_E4M3FN, check, lib, ptr

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16
F16 = torch.float16
ACT_DTYPES = (BF16, F16)   # 16-bit activation formats; fp16 is served by the *_f16 entry points (Hunyuan3D block)


def _act_dtype(t, what):
    """The tensor's dtype if it is one of the two 16-bit activation formats."""
    if t.dtype not in ACT_DTYPES:
        raise TypeError(f"{what}: expected bfloat16 or float16, got {t.dtype}")
    return t.dtype


def _stream(t):
    return torch.cuda.current_stream(t.device).cuda_stream


def _need_hip(t, what, dtype=None):
    if not t.is_cuda:
        raise RuntimeError(f"{what}: tensor is on {t.device}; comfyui_amd only computes on a HIP device "
                           "(there is no CPU path)")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{what}: expected {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{what}: tensor must be contiguous")


def weight_dtype_code(dtype):
    if dtype == BF16:
        return W_BF16
    if dtype == FP8:
        return W_E4M3FN
    if dtype == F16:
        return _lib.W_F16      # hdmoe_linear_bias only
    raise TypeError(f"unsupported weight dtype {dtype}: the HIP path takes bfloat16 or float8_e4m3fn weights")


def gate_top2(x2d, gate_w):
    """MoEGate scoring + top-2 on the device. x2d [T,D] bf16 (or fp16), gate_w [E,D] of the same dtype
    -> topk_idx int32 [T,2], topk_weight [T,2] of that dtype."""
    dt = _act_dtype(x2d, "gate_top2 x")
    _need_hip(x2d, "gate_top2 x", dt)
    _need_hip(gate_w, "gate_top2 gate weight", dt)
    T, D = x2d.shape
    E = gate_w.shape[0]
    if gate_w.shape[1] != D:
        raise ValueError(f"gate weight {tuple(gate_w.shape)} does not match hidden size {D}")
    idx = torch.empty((T, 2), dtype=torch.int32, device=x2d.device)
    w = torch.empty((T, 2), dtype=dt, device=x2d.device)
    fn = lib.hdmoe_gate_top2 if dt == BF16 else lib.hdmoe_gate_top2_f16
    check(fn(ptr(x2d), ptr(gate_w), T, D, E, ptr(idx), ptr(w), _stream(x2d)))
    return idx, w


def renorm_top2(topk_weight):
    """topk_weight / (topk_weight.sum(-1, keepdim=True) + 1e-20) for the [T, 2] bf16 gate weights."""
    _need_hip(topk_weight, "renorm_top2 topk_weight", BF16)
    if topk_weight.dim() != 2 or topk_weight.shape[1] != 2 or not topk_weight.is_contiguous():
        raise ValueError("renorm_top2: expected a contiguous [T, 2] tensor")
    out = torch.empty_like(topk_weight)
    if topk_weight.shape[0] == 0:
        return out
    check(lib.hdmoe_renorm_top2_bf16(ptr(topk_weight), topk_weight.shape[0], ptr(out), _stream(topk_weight)))
    return out


def dispatch(topk_idx, E):
    """Stable permutation of the flat slots by expert.
    -> counts [E], offsets [E+1], perm [2T], inv_perm [2T] (int32, device)."""
    _need_hip(topk_idx, "dispatch topk_idx", torch.int32)
    T = topk_idx.shape[0]
    dev = topk_idx.device
    counts = torch.empty(E, dtype=torch.int32, device=dev)
    offsets = torch.empty(E + 1, dtype=torch.int32, device=dev)
    perm = torch.empty(2 * T, dtype=torch.int32, device=dev)
    inv = torch.empty(2 * T, dtype=torch.int32, device=dev)
    nbytes = lib.hdmoe_dispatch_workspace_bytes(T, E)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=dev)
    check(lib.hdmoe_dispatch(ptr(topk_idx), T, E, ptr(counts), ptr(offsets), ptr(perm), ptr(inv), ptr(ws), nbytes,
                             _stream(topk_idx)))
    return counts, offsets, perm, inv


def _scale_ptr(s, device, what):
    if s is None:
        return None
    if s.device != device or s.dtype != torch.float32 or s.numel() != 1:
        raise ValueError(f"{what} must be an fp32 scalar tensor on {device}")
    return s.data_ptr()


def quant_fp8(x, scale_input):
    """fp8_linear's activation cast: x bf16 [..., D] -> float8_e4m3fn, same shape."""
    _need_hip(x, "quant_fp8 x", BF16)
    D = x.shape[-1]
    out = torch.empty(x.shape, dtype=FP8, device=x.device)
    check(lib.hdmoe_quant_fp8(ptr(x), x.numel() // D, D, _scale_ptr(scale_input, x.device, "scale_input"), ptr(out),
                              _stream(x)))
    return out


def quant_permute_fp8(x2d, perm, offsets, scale_inputs):
    """Gather rows by perm and quantise each with its expert's scale_input. -> [2T,D] fp8."""
    _need_hip(x2d, "quant_permute_fp8 x", BF16)
    T, D = x2d.shape
    E = len(scale_inputs)
    arr = (ctypes.c_void_p * E)(*[_scale_ptr(s, x2d.device, "scale_input") for s in scale_inputs])
    out = torch.empty((2 * T, D), dtype=FP8, device=x2d.device)
    check(lib.hdmoe_quant_permute_fp8(ptr(x2d), ptr(perm), ptr(offsets), T, D, E, arr, ptr(out), _stream(x2d)))
    return out


def permute_bf16(x2d, perm):
    """a[r] = x[perm[r] / 2]; rows are copied as bytes, so fp16 rows go through the same kernel."""
    dt = _act_dtype(x2d, "permute_bf16 x")
    _need_hip(x2d, "permute_bf16 x", dt)
    T, D = x2d.shape
    out = torch.empty((2 * T, D), dtype=dt, device=x2d.device)
    check(lib.hdmoe_permute_bf16(ptr(x2d), ptr(perm), T, D, ptr(out), _stream(x2d)))
    return out


def linear(a2d, weight, scale_weight=None, scale_input=None, bias=None):
    """a2d [rows,K] (fp8 for fp8 weights, bf16 for bf16 weights, fp16 for fp16 weights) x weight [N,K]^T (+ bias [N])
    -> [rows,N] bf16 (fp16 for fp16 weights); the bias joins the fp32 result before the one rounding."""
    code = weight_dtype_code(weight.dtype)
    _need_hip(a2d, "linear activations", weight.dtype)
    _need_hip(weight, "linear weight")
    rows, K = a2d.shape
    N = weight.shape[0]
    if weight.shape[1] != K:
        raise ValueError(f"linear: activations [{rows},{K}] do not match weight {tuple(weight.shape)}")
    out_dtype = F16 if weight.dtype == F16 else BF16
    if bias is not None:
        _need_hip(bias, "linear bias", out_dtype)
        if bias.shape != (N,) or not bias.is_contiguous():
            raise ValueError(f"linear: bias {tuple(bias.shape)} does not match {N} output features")
    out = torch.empty((rows, N), dtype=out_dtype, device=a2d.device)
    check(lib.hdmoe_linear_bias(code, ptr(a2d), rows, K, N, ptr(weight),
                                _scale_ptr(scale_weight, a2d.device, "scale_weight"),
                                _scale_ptr(scale_input, a2d.device, "scale_input"), ptr(bias), ptr(out), _stream(a2d)))
    return out


def silu_mul(a, b):
    _need_hip(a, "silu_mul a", BF16)
    _need_hip(b, "silu_mul b", BF16)
    if a.shape != b.shape:
        raise ValueError("silu_mul: shape mismatch")
    out = torch.empty_like(a)
    check(lib.hdmoe_silu_mul_bf16(ptr(a), ptr(b), a.numel(), ptr(out), _stream(a)))
    return out


def gelu(x):
    """F.gelu (erf form) of a contiguous bf16 or fp16 tensor."""
    dt = _act_dtype(x, "gelu x")
    _need_hip(x, "gelu x", dt)
    out = torch.empty_like(x)
    fn = lib.hdmoe_gelu_bf16 if dt == BF16 else lib.hdmoe_gelu_f16
    check(fn(ptr(x), x.numel(), ptr(out), _stream(x)))
    return out


def scale_to_bf16(src, scale):
    """bf16(bf16(src) * bf16(scale)) for src in fp8 or bf16."""
    code = weight_dtype_code(src.dtype)
    _need_hip(src, "scale_to_bf16 src")
    out = torch.empty(src.shape, dtype=BF16, device=src.device)
    check(lib.hdmoe_scale_to_bf16(code, ptr(src), src.numel(), _scale_ptr(scale, src.device, "scale"), ptr(out),
                                  _stream(src)))
    return out


def combine(y_sorted, inv_perm, topk_weight, shared):
    dt = _act_dtype(y_sorted, "combine y")
    _need_hip(y_sorted, "combine y", dt)
    _need_hip(topk_weight, "combine topk_weight", dt)
    if shared is not None:
        _need_hip(shared, "combine shared", dt)
    T = topk_weight.shape[0]
    D = y_sorted.shape[1]
    out = torch.empty((T, D), dtype=dt, device=y_sorted.device)
    fn = lib.hdmoe_combine if dt == BF16 else lib.hdmoe_combine_f16
    check(fn(ptr(y_sorted), ptr(inv_perm), ptr(topk_weight), ptr(shared), T, D, ptr(out), _stream(y_sorted)))
    return out


def _linear_weights(weight, bias, K, N, what, dtype=BF16):
    _need_hip(weight, f"{what} weight", dtype)
    if tuple(weight.shape) != (N, K):
        raise ValueError(f"{what}: weight shape {tuple(weight.shape)} != ({N}, {K})")
    lw = LinearWeights()
    lw.weight = ptr(weight)
    if bias is not None:
        _need_hip(bias, f"{what} bias", dtype)
        if tuple(bias.shape) != (N,):
            raise ValueError(f"{what}: bias shape {tuple(bias.shape)} != ({N},)")
        lw.bias = ptr(bias)
    return lw


def grouped_linear(a_sorted, offsets, experts, a_static=None, shared=None, act="none"):
    """Linear (+ bias, + erf GELU) of every expert over its row segment of `a_sorted` [rows, K] and, optionally, of
    one more (weight, bias) over all rows of `a_static`, in one launch. experts: list of (weight [N,K], bias [N] or
    None). Returns (out_sorted [rows, N], out_static [rows_static, N] or None)."""
    code = {"none": _lib.ACT_NONE, "gelu": _lib.ACT_GELU}[act]
    dt = _act_dtype(a_sorted, "grouped_linear a")   # bf16, or fp16 throughout
    _need_hip(a_sorted, "grouped_linear a", dt)
    rows, K = a_sorted.shape
    N = experts[0][0].shape[0] if experts else shared[0].shape[0]
    E = len(experts)
    arr = (LinearWeights * max(E, 1))(*[_linear_weights(w, b, K, N, f"grouped_linear expert {i}", dt)
                                        for i, (w, b) in enumerate(experts)])
    out = torch.empty((rows, N), dtype=dt, device=a_sorted.device)
    out_static, sh, rows_static = None, None, 0
    if shared is not None:
        _need_hip(a_static, "grouped_linear a_static", dt)
        rows_static = a_static.shape[0]
        sh = _linear_weights(shared[0], shared[1], K, N, "grouped_linear shared", dt)
        out_static = torch.empty((rows_static, N), dtype=dt, device=a_sorted.device)
    fn = lib.hdmoe_grouped_linear if dt == BF16 else lib.hdmoe_grouped_linear_f16
    check(fn(ptr(a_sorted), ptr(offsets), rows, E, arr, ptr(out), ptr(a_static), rows_static,
                                   ctypes.byref(sh) if sh is not None else None, ptr(out_static), K, N, code,
                                   _stream(a_sorted)))
    return out, out_static


def grouped_linear_tokens(x2d, perm, offsets, experts, shared=None, act="none"):
    """The first Linear (+ bias, + erf GELU) of every expert on the rows of `x2d` [T, K] its segment selects through
    the dispatch permutation (sorted row r = token perm[r] // 2; nothing is copied into expert order), and of
    `shared` (weight, bias) on all T rows, in one launch. Returns (out_sorted [2T, N], out_shared [T, N] or None)."""
    code = {"none": _lib.ACT_NONE, "gelu": _lib.ACT_GELU}[act]
    dt = _act_dtype(x2d, "grouped_linear_tokens x")
    _need_hip(x2d, "grouped_linear_tokens x", dt)
    T, K = x2d.shape
    N = experts[0][0].shape[0]
    E = len(experts)
    arr = (LinearWeights * E)(*[_linear_weights(w, b, K, N, f"grouped_linear_tokens expert {i}", dt)
                                for i, (w, b) in enumerate(experts)])
    out = torch.empty((T * _lib.TOPK, N), dtype=dt, device=x2d.device)
    out_shared, sh = None, None
    if shared is not None:
        sh = _linear_weights(shared[0], shared[1], K, N, "grouped_linear_tokens shared", dt)
        out_shared = torch.empty((T, N), dtype=dt, device=x2d.device)
    check(lib.hdmoe_grouped_linear_tokens(_lib.W_BF16 if dt == BF16 else _lib.W_F16, ptr(x2d), T, ptr(perm), ptr(offsets), E,
                                          arr, ptr(out), ctypes.byref(sh) if sh is not None else None, ptr(out_shared),
                                          K, N, code, _stream(x2d)))
    return out, out_shared


def stochastic_round_e4m3fn(weight, scale=None, seed=0):
    """weight (fp32 or bf16, HIP) / scale (fp32 scalar tensor or None) -> float8_e4m3fn by stochastic rounding
    (comfy/float.py:14-67 behind comfy/ops.py:419-426), one kernel."""
    _need_hip(weight, "stochastic_round_e4m3fn weight")
    if weight.dtype == torch.float32:
        code = _lib.SRC_F32
    elif weight.dtype == BF16:
        code = _lib.SRC_BF16
    else:
        raise TypeError(f"stochastic_round_e4m3fn: expected float32 or bfloat16, got {weight.dtype}")
    out = torch.empty(weight.shape, dtype=FP8, device=weight.device)
    check(lib.hdmoe_stochastic_round_e4m3fn(code, ptr(weight), weight.numel(),
                                            _scale_ptr(scale, weight.device, "stochastic_round_e4m3fn scale"),
                                            int(seed) & 0xFFFFFFFFFFFFFFFF, ptr(out), _stream(weight)))
    return out


def _per_batch(t, what, D, device):
    """[B, D] (or [B, 1, D]) bf16 modulation rows -> contiguous [B, D]."""
    _need_hip(t, what, BF16)
    if t.dim() == 3 and t.shape[1] == 1:
        t = t[:, 0]
    if t.dim() != 2 or t.shape[1] != D or not t.is_contiguous():
        raise ValueError(f"{what}: expected a contiguous [batch, {D}] tensor, got {tuple(t.shape)}")
    return t


def ln_modulate(x2d, scale, shift, tokens_per_batch, eps=1e-6):
    """bf16 LayerNorm(x) * (1 + scale) + shift with scale/shift one row per batch item
    (comfy/ldm/hidream/model.py:430-431, 516-517)."""
    _need_hip(x2d, "ln_modulate x", BF16)
    T, D = x2d.shape
    scale = _per_batch(scale, "ln_modulate scale", D, x2d.device)
    shift = _per_batch(shift, "ln_modulate shift", D, x2d.device)
    if tokens_per_batch <= 0 or T != scale.shape[0] * tokens_per_batch or shift.shape != scale.shape:
        raise ValueError(f"ln_modulate: T={T} is not batch={scale.shape[0]} x tokens_per_batch={tokens_per_batch}")
    out = torch.empty_like(x2d)
    check(lib.hdmoe_ln_modulate_bf16(ptr(x2d), ptr(scale), ptr(shift), T, D, tokens_per_batch, eps, ptr(out),
                                     _stream(x2d)))
    return out


def combine_gated_residual(y_sorted, inv_perm, topk_weight, shared, gate, residual, tokens_per_batch):
    """combine(), then gate * y + residual (comfy/ldm/hidream/model.py:432-433, 518-523)."""
    _need_hip(y_sorted, "combine y", BF16)
    _need_hip(topk_weight, "combine topk_weight", BF16)
    _need_hip(residual, "combine residual", BF16)
    T = topk_weight.shape[0]
    D = y_sorted.shape[1]
    gate = _per_batch(gate, "combine gate", D, y_sorted.device)
    if tokens_per_batch <= 0 or T != gate.shape[0] * tokens_per_batch or tuple(residual.shape) != (T, D):
        raise ValueError(f"combine_gated_residual: T={T}, batch={gate.shape[0]}, tokens_per_batch={tokens_per_batch}")
    out = torch.empty((T, D), dtype=BF16, device=y_sorted.device)
    check(lib.hdmoe_combine_gated_residual(ptr(y_sorted), ptr(inv_perm), ptr(topk_weight), ptr(shared), ptr(gate),
                                           ptr(residual), tokens_per_batch, T, D, ptr(out), _stream(y_sorted)))
    return out


def gated_residual(y2d, gate, residual2d, tokens_per_batch):
    """gate * y + residual behind a dense feed-forward (comfy/ldm/hidream/model.py:519-523)."""
    _need_hip(y2d, "gated_residual y", BF16)
    _need_hip(residual2d, "gated_residual residual", BF16)
    T, D = y2d.shape
    gate = _per_batch(gate, "gated_residual gate", D, y2d.device)
    if tokens_per_batch <= 0 or T != gate.shape[0] * tokens_per_batch or tuple(residual2d.shape) != (T, D):
        raise ValueError(f"gated_residual: T={T}, batch={gate.shape[0]}, tokens_per_batch={tokens_per_batch}")
    out = torch.empty_like(y2d)
    check(lib.hdmoe_gated_residual_bf16(ptr(y2d), ptr(gate), ptr(residual2d), tokens_per_batch, T, D, ptr(out),
                                        _stream(y2d)))
    return out


def make_ffn_weights(w1, w2, w3, scales=None, same_scale_in13=False):
    """Fill an hdmoe_ffn_weights. scales: dict with optional fp32 scalar tensors
    scale_w1/2/3 and scale_in1/2/3 (fp8 only). same_scale_in13: the caller has checked that scale_in1 and
    scale_in3, two different tensors, hold the same value (the library refuses two different pointers otherwise)."""
    fw = FfnWeights()
    fw.w1, fw.w2, fw.w3 = ptr(w1), ptr(w2), ptr(w3)
    if scales:
        for k, v in scales.items():
            setattr(fw, k, ptr(v))
    fw.same_scale_in13 = 1 if same_scale_in13 else 0
    return fw


def grouped_swiglu(a, offsets, experts, H):
    """experts: list of FfnWeights. a [2T,D] -> h [2T,H] (same element type as a)."""
    code = weight_dtype_code(a.dtype)
    _need_hip(a, "grouped_swiglu a")
    rows, D = a.shape
    E = len(experts)
    arr = (FfnWeights * E)(*experts)
    h = torch.empty((rows, H), dtype=a.dtype, device=a.device)
    check(lib.hdmoe_grouped_swiglu(code, ptr(a), ptr(offsets), rows, E, D, H, arr, ptr(h), _stream(a)))
    return h


def grouped_down(h, offsets, experts, D):
    code = weight_dtype_code(h.dtype)
    _need_hip(h, "grouped_down h")
    rows, H = h.shape
    E = len(experts)
    arr = (FfnWeights * E)(*experts)
    y = torch.empty((rows, D), dtype=BF16, device=h.device)
    check(lib.hdmoe_grouped_down(code, ptr(h), ptr(offsets), rows, E, H, D, arr, ptr(y), _stream(h)))
    return y


def ffn_swiglu(x2d, weights, H, weight_dtype):
    """One dense SwiGLU feed-forward as three enqueues. weights: FfnWeights. x2d [rows,D] bf16 -> [rows,D] bf16."""
    _need_hip(x2d, "ffn_swiglu x", BF16)
    rows, D = x2d.shape
    code = weight_dtype_code(weight_dtype)
    nbytes = lib.hdmoe_ffn_workspace_bytes(rows, D, H, code)
    ws = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=x2d.device)
    out = torch.empty((rows, D), dtype=BF16, device=x2d.device)
    fw = FfnWeights.from_buffer_copy(weights)
    check(lib.hdmoe_ffn_swiglu(code, ptr(x2d), rows, D, H, ctypes.byref(fw), ptr(out), ptr(ws), ws.numel(),
                               _stream(x2d)))
    return out


def layer_layout(T, D, H, Hs, E, code):
    lay = LayerLayout()
    check(lib.hdmoe_layer_layout_get(T, D, H, Hs, E, code, ctypes.byref(lay)))
    return lay


def moe_ffn(x2d, gate_w, experts, shared, H, Hs, weight_dtype, out=None, workspace=None, want_routing=False,
            stage_events=None, modulation=None, tokens_per_batch=None, ln_eps=1e-6, uniform_scale_in=False,
            scale_check=None, fixed_k_cut=False):
    """The whole layer as one enqueue. experts: list of FfnWeights, shared: FfnWeights or None.
    modulation=(shift, scale, gate), each [B, D] bf16, turns the call into the block's feed-forward branch:
    out = x + gate * layer(LayerNorm(x) * (1 + scale) + shift), with T == B * tokens_per_batch.
    uniform_scale_in: accepted and not used (the casting kernel compares the scale_input values on the device and
    casts the tokens once when they agree).
    fixed_k_cut: the K cut of the down projection (small token counts) is taken from the sizes alone instead of from
    the segment sizes of the call, so that a row's bytes do not depend on the routing of the other rows.
    scale_check: optional pinned int32 tensor of one element that the casting kernel sets to 1 when w1 and w3 of a
    feed-forward turn out to cast the tokens differently (the output is then NaN).
    Returns out [T,D] bf16 (and topk_idx int32, topk_weight bf16 when want_routing)."""
    _need_hip(x2d, "moe_ffn x", BF16)
    _need_hip(gate_w, "moe_ffn gate weight", BF16)
    T, D = x2d.shape
    E = len(experts)
    code = weight_dtype_code(weight_dtype)
    nbytes = lib.hdmoe_layer_workspace_bytes(T, D, H, Hs if shared is not None else 0, E, code)
    if nbytes == 0 and T > 0:
        raise _lib.HdmoeError(_lib.lib.hdmoe_layer_layout_get(T, D, H, Hs, E, code, ctypes.byref(LayerLayout())),
                              lib.hdmoe_last_error().decode())
    if workspace is None or workspace.numel() < nbytes:
        workspace = torch.empty(max(nbytes, 256), dtype=torch.uint8, device=x2d.device)
    if out is None:
        out = torch.empty((T, D), dtype=BF16, device=x2d.device)
    args = LayerArgs()
    args.T, args.D, args.H, args.Hs, args.E, args.weight_dtype = T, D, H, (Hs if shared is not None else 0), E, code
    args.x, args.gate_w = ptr(x2d), ptr(gate_w)
    arr = (FfnWeights * E)(*experts)
    args.experts = arr
    sh = None
    if shared is not None:
        sh = FfnWeights.from_buffer_copy(shared)
        args.shared = ctypes.pointer(sh)
    args.out, args.workspace, args.workspace_bytes = ptr(out), ptr(workspace), workspace.numel()
    args.uniform_scale_in = 1 if uniform_scale_in else 0
    args.fixed_k_cut = 1 if fixed_k_cut else 0
    if scale_check is not None:
        if scale_check.dtype != torch.int32 or scale_check.numel() < 1 or not (scale_check.is_cuda or scale_check.is_pinned()):
            raise TypeError("moe_ffn: scale_check must be an int32 tensor on the device or in pinned host memory")
        args.scale_check = ptr(scale_check)
    if modulation is not None:
        shift, scale, gate = (_per_batch(m, "moe_ffn modulation", D, x2d.device) for m in modulation)
        if not tokens_per_batch or T != shift.shape[0] * tokens_per_batch or not (shift.shape == scale.shape == gate.shape):
            raise ValueError(f"moe_ffn: T={T} is not batch={shift.shape[0]} x tokens_per_batch={tokens_per_batch}")
        args.mod_shift, args.mod_scale, args.mod_gate = ptr(shift), ptr(scale), ptr(gate)
        args.tokens_per_batch, args.ln_eps = tokens_per_batch, ln_eps
    idx = tw = None
    if want_routing:
        idx = torch.empty((T, 2), dtype=torch.int32, device=x2d.device)
        tw = torch.empty((T, 2), dtype=BF16, device=x2d.device)
        args.topk_idx, args.topk_weight = ptr(idx), ptr(tw)
    if stage_events is not None:
        # sequence of NUM_STAGES + 1 hipEvent_t handles (ints) created by the caller
        ev = (ctypes.c_void_p * (_lib.NUM_STAGES + 1))(*stage_events)
        args.stage_events = ev
    check(lib.hdmoe_moe_ffn(ctypes.byref(args), _stream(x2d)))
    # the workspace must outlive the enqueued kernels: torch's caching allocator keeps a freed block
    # tied to the stream it was allocated on, so releasing it here is safe for work on that stream
    if want_routing:
        return out, idx, tw
    return out
