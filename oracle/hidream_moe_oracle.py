"""TEST INFRASTRUCTURE ONLY -- CPU oracle for the HiDream MoE SwiGLU feed-forward.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; nothing under comfyui_amd/ does.

It restates, with torch CPU tensors as the array library (the reference itself is
torch code; torch 2.10.0 is what this image carries, requirements.txt:4 leaves it
unpinned), the dataflow of these reference functions (paths under /root/reference):

  comfy/ldm/hidream/model.py:237-238   FeedForwardSwiGLU.forward      -> ffn_swiglu
  comfy/ldm/hidream/model.py:263-283   MoEGate.forward                -> gate_torch / gate_fixed_order
  comfy/ldm/hidream/model.py:307-325   MOEFeedForwardSwiGLU.forward   -> moe_forward
  comfy/ops.py:103-115, 283-284        (manual_cast) Linear           -> Linear mode "plain"
  comfy/ops.py:399-410                 scaled_fp8 Linear, upcast path -> Linear mode "upcast"
  comfy/ops.py:314-358                 fp8_linear                     -> Linear mode "fp8mm"

The reference has no golden vectors, known-answer tests or fixtures for any of
these (its tests never touch comfy.ops or hidream), so every function is pinned by
tests/test_oracle_*.py against closed forms, brute force on tiny inputs, dense
(every expert on every token) evaluation, invariants, and torch library routines.

Top-2 selection: the reference calls torch.topk(sorted=False), whose tie choice is
an implementation detail of torch; the contract here is "larger score first, ties
to the lower expert index", i.e. the first two entries of a stable descending sort.
"""
import ctypes
import os

import numpy as np
import torch
import torch.nn.functional as F

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def _lib():
    """The C part of the oracle (moe_ref.c), built by `make -C oracle`."""
    global _LIB
    if _LIB is None:
        path = os.path.join(_HERE, "libhdmoe_oracle.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} missing: run `make -C oracle` (or __graft_entry__.build())")
        lib = ctypes.CDLL(path)
        lib.ref_gate_top2.restype = ctypes.c_int
        lib.ref_gate_top2_f16.restype = ctypes.c_int
        lib.ref_f16_decode.restype = None
        lib.ref_f16_encode.restype = None
        lib.ref_dispatch.restype = ctypes.c_int
        lib.ref_combine.restype = None
        lib.ref_ln_modulate.restype = ctypes.c_int
        lib.ref_ln_modulate.argtypes = [ctypes.c_void_p] * 3 + [ctypes.c_int] * 3 + [ctypes.c_float, ctypes.c_void_p]
        lib.ref_gated_residual.restype = None
        lib.ref_philox4x32_10.restype = None
        lib.ref_stochastic_round_e4m3fn.restype = None
        lib.ref_stochastic_round_e4m3fn.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_uint64,
                                                    ctypes.c_int, ctypes.c_void_p]
        lib.ref_e4m3fn_encode.restype = None
        lib.ref_e4m3fn_decode_table.restype = None
        _LIB = lib
    return _LIB


def _p(t):
    return ctypes.c_void_p(t.data_ptr())


# --------------------------------------------------------------------------- fp8

def e4m3fn_decode_table():
    out = torch.empty(256, dtype=torch.float32)
    _lib().ref_e4m3fn_decode_table(_p(out))
    return out


def e4m3fn_encode(x_f32):
    """fp32 -> e4m3fn bytes (uint8): RNE, |v|>464 -> NaN (ops.py:340,343 `.to(dtype)`)."""
    x = x_f32.detach().to(torch.float32).contiguous()
    out = torch.empty(x.shape, dtype=torch.uint8)
    _lib().ref_e4m3fn_encode(_p(x), _p(out), ctypes.c_int64(x.numel()))
    return out


def e4m3fn_decode(b_u8):
    return e4m3fn_decode_table()[b_u8.long()]


def quantize_weight_per_tensor(w_f32):
    """Per-tensor weight quantisation of the scaled-fp8 benchmark layers: scale_weight = amax/448, W8 = (W/scale_weight) -> e4m3fn.
    Returns (W8 as torch.float8_e4m3fn, scale_weight fp32 scalar tensor)."""
    w = w_f32.to(torch.float32)
    s = (w.abs().amax() / 448.0).to(torch.float32)
    w8 = (w / s).to(torch.float8_e4m3fn)
    return w8, s


# -------------------------------------------------------------------------- gate

def f16_decode(bits_u16):
    """fp16 bit patterns (int16/uint16 tensor) -> fp32 by the format's definition (moe_ref.c f16_to_f32)."""
    src = bits_u16.contiguous()
    out = torch.empty(src.shape, dtype=torch.float32)
    _lib().ref_f16_decode(_p(src), _p(out), ctypes.c_int64(src.numel()))
    return out


def f16_encode(values_f32):
    """fp32 -> fp16 bit patterns (int16), round to nearest even, overflow to infinity (moe_ref.c f32_to_f16)."""
    src = values_f32.float().contiguous()
    out = torch.empty(src.shape, dtype=torch.int16)
    _lib().ref_f16_encode(_p(src), _p(out), ctypes.c_int64(src.numel()))
    return out


def top2_lowest_index(scores):
    """First two columns of a stable descending sort: larger score first, ties -> lower index."""
    order = torch.sort(scores.float(), dim=-1, descending=True, stable=True).indices
    idx = order[:, :2].contiguous()
    return idx, torch.gather(scores, 1, idx)


def gate_torch(x2d, wg):
    """model.py:267-275 with torch's own kernels at x's dtype (bf16 or fp32):
    F.linear -> softmax -> top-2. Returns idx int64 [T,2], weight [T,2], logits, scores."""
    logits = F.linear(x2d, wg.to(x2d.dtype), None)
    scores = logits.softmax(dim=-1)
    idx, w = top2_lowest_index(scores)
    return idx, w, logits, scores


def gate_fixed_order(x2d_bf16, wg_bf16):
    """Same computation with the one fixed fp32 summation order and exp() of moe_ref.c
    (what the HIP gate kernel is compared with bit for bit).
    Returns idx int32 [T,2], weight bf16 [T,2], logits bf16 [T,E], scores bf16 [T,E]. fp16 inputs: the same with
    every tensor and the two roundings in fp16 (the Hunyuan3D block's other dtype)."""
    x = x2d_bf16.contiguous()
    wg = wg_bf16.contiguous()
    assert x.dtype in (torch.bfloat16, torch.float16) and wg.dtype == x.dtype
    T, D = x.shape
    E = wg.shape[0]
    idx = torch.empty((T, 2), dtype=torch.int32)
    w = torch.empty((T, 2), dtype=x.dtype)
    logits = torch.empty((T, E), dtype=x.dtype)
    scores = torch.empty((T, E), dtype=x.dtype)
    fn = _lib().ref_gate_top2 if x.dtype == torch.bfloat16 else _lib().ref_gate_top2_f16
    rc = fn(_p(x), _p(wg), T, D, E, _p(idx), _p(w), _p(logits), _p(scores))
    if rc != 0:
        raise ValueError("ref_gate_top2: bad arguments")
    return idx, w, logits, scores


# ---------------------------------------------------------------------- dispatch

def dispatch(topk_idx, E):
    """Stable counting sort of the flat expert ids (model.py:313-318).
    Returns counts[E], offsets[E+1], perm[2T], inv_perm[2T] (int32)."""
    flat = topk_idx.reshape(-1).to(torch.int32).contiguous()
    n = flat.numel()
    counts = torch.empty(E, dtype=torch.int32)
    offsets = torch.empty(E + 1, dtype=torch.int32)
    perm = torch.empty(n, dtype=torch.int32)
    inv = torch.empty(n, dtype=torch.int32)
    rc = _lib().ref_dispatch(_p(flat), ctypes.c_int64(n), E, _p(counts), _p(offsets), _p(perm), _p(inv))
    if rc != 0:
        raise ValueError("ref_dispatch: expert id out of range")
    return counts, offsets, perm, inv


def combine_c(y_sorted_bf16, inv_perm, w_bf16, shared_bf16):
    """C restatement of model.py:319,324 at bf16 (see moe_ref.c ref_combine)."""
    T = w_bf16.shape[0]
    D = y_sorted_bf16.shape[1]
    out = torch.empty((T, D), dtype=torch.bfloat16)
    _lib().ref_combine(_p(y_sorted_bf16.contiguous()), _p(inv_perm.contiguous()), _p(w_bf16.contiguous()),
                       _p(shared_bf16.contiguous()) if shared_bf16 is not None else None, T, D, _p(out))
    return out


# ------------------------------------------------------------------------ linear

class LinearParams:
    """One reference Linear: weight [out,in] (bf16/fp32, or float8_e4m3fn with scale_weight and optional
    scale_input fp32 scalars, ops.py:388-397) and an optional bias [out]."""

    def __init__(self, weight, scale_weight=None, scale_input=None, bias=None):
        self.weight = weight
        self.scale_weight = scale_weight
        self.scale_input = scale_input
        self.bias = bias


def oracle_params(state_dict, num_experts):
    """Module state dict (bf16, or scaled fp8 with .scale_weight/.scale_input) -> params for moe_forward."""
    def lin(prefix):
        return LinearParams(state_dict[prefix + ".weight"], state_dict.get(prefix + ".scale_weight"),
                            state_dict.get(prefix + ".scale_input"))

    def ffn(prefix):
        return (lin(prefix + "w1"), lin(prefix + "w2"), lin(prefix + "w3"))

    return dict(gate=state_dict["gate.weight"], experts=[ffn(f"experts.{e}.") for e in range(num_experts)],
                shared=ffn("shared_experts."))


def linear(x, p, mode):
    """mode "plain":  F.linear at x.dtype with the weight cast to x.dtype (ops.py:107-109).
    mode "upcast": scaled-fp8 Linear without fp8 matmul (ops.py:405-410).
    mode "fp8mm":  fp8_linear (ops.py:314-358): quantise x (x * (1/scale_input).to(x.dtype) -> e4m3fn,
                   or clamp +-448 when scale_input is None), fp8 x fp8 products accumulated in fp32,
                   times scale_input*scale_weight, rounded to x.dtype. Products of two e4m3 values are
                   exact in fp32, so an fp32 matmul of the decoded operands is the same contraction.
                   A bias (cast to x.dtype, ops.py:329) goes into the scaled matrix multiply (ops.py:345-346),
                   which adds it to the scaled fp32 result before the one rounding (checked against
                   torch._scaled_mm itself in the tests).
    Modes "plain" and "upcast" with a bias: F.linear's own bias argument."""
    bias = getattr(p, "bias", None)
    if bias is not None:
        bias = bias.to(x.dtype)
    if mode == "plain":
        return F.linear(x, p.weight.to(x.dtype), bias)
    if mode == "upcast":
        w = p.weight.to(x.dtype)
        s = p.scale_weight.to(x.dtype)
        if w.numel() < x.numel():
            return F.linear(x, w * s, bias)
        return F.linear(x * s, w, bias)
    if mode == "fp8mm":
        assert p.weight.dtype == torch.float8_e4m3fn
        if p.scale_input is None:
            s_in = torch.ones((), dtype=torch.float32)
            xq = torch.clamp(x, min=-448, max=448).to(torch.float8_e4m3fn)
        else:
            s_in = p.scale_input.to(torch.float32)
            xq = (x * (1.0 / s_in).to(x.dtype)).to(torch.float8_e4m3fn)
        acc = xq.to(torch.float32) @ p.weight.to(torch.float32).t()
        acc = acc * (s_in * p.scale_weight.to(torch.float32))
        if bias is not None:
            acc = acc + bias.to(torch.float32)
        return acc.to(x.dtype)
    raise ValueError(mode)


def ffn_swiglu(x, ffn, mode):
    """model.py:238: w2(silu(w1 x) * w3 x); every op rounds to x.dtype as torch does."""
    w1, w2, w3 = ffn
    return linear(F.silu(linear(x, w1, mode)) * linear(x, w3, mode), w2, mode)


# ------------------------------------------------------------------------- layer

def moe_forward(x, params, mode, gate_result=None):
    """model.py:307-325, literally: gate, repeat_interleave, boolean-mask gather per expert,
    weighted sum over the K slots, plus the shared expert.
    params: dict(gate=Wg [E,D], experts=[(w1,w2,w3)]*E, shared=(w1,w2,w3)) of LinearParams.
    gate_result: optional (topk_idx, topk_weight) to reuse a routing decision (e.g. the GPU's)."""
    wtype = x.dtype
    orig_shape = x.shape
    x2 = x.reshape(-1, x.shape[-1])
    if gate_result is None:
        topk_idx, topk_weight, _, _ = gate_torch(x2, params["gate"])
    else:
        topk_idx, topk_weight = gate_result
        topk_idx = topk_idx.long()
        topk_weight = topk_weight.to(wtype)
    K = topk_idx.shape[1]
    flat = topk_idx.reshape(-1)
    xr = x2.repeat_interleave(K, dim=0)
    y = torch.zeros_like(xr)
    for i, ffn in enumerate(params["experts"]):
        m = flat == i
        if bool(m.any()):
            y[m] = ffn_swiglu(xr[m], ffn, mode).to(wtype)
    y = (y.view(*topk_weight.shape, -1) * topk_weight.unsqueeze(-1)).sum(dim=1)
    y = y.view(*orig_shape).to(wtype)
    return y + ffn_swiglu(x, params["shared"], mode)


# --------------------------------------------- Hunyuan3D-2.1 MoEBlock (hunyuandit.py:8-188)

def linear_bias(x, weight, bias):
    """operations.Linear with bias at x.dtype: the contraction and the bias add in fp32, one rounding to x.dtype
    (what a GEMM with a bias epilogue does; torch's own bf16 F.linear agrees to one step, see the tests)."""
    acc = x.float() @ weight.float().t()
    if bias is not None:
        acc = acc + bias.float()
    return acc.to(x.dtype)


def gelu_feed_forward(x, ff):
    """hunyuandit.py:28-50: Linear -> F.gelu (erf form) -> Dropout(0) -> Linear. ff = (w_in, b_in, w_out, b_out), or
    (LinearParams, LinearParams, mode) for Linears of the operation classes (`linear` above)."""
    if len(ff) == 3:
        p_in, p_out, mode = ff
        return linear(F.gelu(linear(x, p_in, mode)), p_out, mode)
    w_in, b_in, w_out, b_out = ff
    return linear_bias(F.gelu(linear_bias(x, w_in, b_in)), w_out, b_out)


def hunyuan_moe_block(x, params, gate_result=None):
    """hunyuandit.py:131-187 (inference branch), literally: gate, argsort of the flat expert ids, per expert the
    tokens in sorted order, output times the routing weight, index_add_ into a zero cache in expert order, plus
    the shared expert. params: dict(gate=Wg [E,D], experts=[(w_in,b_in,w_out,b_out)]*E, shared=(...))."""
    orig_shape = x.shape
    x2 = x.reshape(-1, x.shape[-1])
    if gate_result is None:
        topk_idx, topk_weight, _, _ = gate_torch(x2, params["gate"])
    else:
        topk_idx, topk_weight = gate_result
        topk_idx = topk_idx.long()
        topk_weight = topk_weight.to(x.dtype)
    top_k = topk_idx.shape[1]
    flat_idx = topk_idx.reshape(-1)
    flat_w = topk_weight.reshape(-1, 1)
    cache = torch.zeros_like(x2)
    idxs = flat_idx.argsort(stable=True)
    ends = flat_idx.bincount(minlength=len(params["experts"])).cumsum(0)
    token_idxs = idxs // top_k
    for i, end in enumerate(ends.tolist()):
        start = 0 if i == 0 else int(ends[i - 1])
        if start == end:
            continue
        tok = token_idxs[start:end]
        out = gelu_feed_forward(x2[tok], params["experts"][i])
        out.mul_(flat_w[idxs[start:end]])
        cache.index_add_(0, tok, out)
    return cache.view(*orig_shape) + gelu_feed_forward(x, params["shared"])


def hunyuan_moe_block_dense(x, params, topk_idx, topk_weight):
    """Brute force used to pin hunyuan_moe_block: every expert on every token, selected by mask."""
    x2 = x.reshape(-1, x.shape[-1])
    outs = torch.stack([gelu_feed_forward(x2, ff) for ff in params["experts"]], dim=0)   # [E,T,D]
    T = x2.shape[0]
    sel = outs[topk_idx.long().t(), torch.arange(T).unsqueeze(0)]                        # [K,T,D]
    y = (sel.permute(1, 0, 2) * topk_weight.to(x.dtype).unsqueeze(-1)).sum(dim=1)
    return y.view(x.shape).to(x.dtype) + gelu_feed_forward(x, params["shared"])


def hunyuan_params(state_dict, num_experts):
    """MoEBlock state dict (keys experts.N.net.0.proj.*, experts.N.net.2.*, shared_experts.*, gate.weight)."""
    def ff(prefix):
        return (state_dict[prefix + "net.0.proj.weight"], state_dict.get(prefix + "net.0.proj.bias"),
                state_dict[prefix + "net.2.weight"], state_dict.get(prefix + "net.2.bias"))
    return dict(gate=state_dict["gate.weight"], experts=[ff(f"experts.{i}.") for i in range(num_experts)],
                shared=ff("shared_experts."))


# ------------------------------------------------------------- weight maintenance

def philox4x32_10(ctr, key):
    """The checker's Philox4x32-10: 4 counter words, 2 key words -> 4 output words."""
    c = (ctypes.c_uint32 * 4)(*ctr)
    k = (ctypes.c_uint32 * 2)(*key)
    o = (ctypes.c_uint32 * 4)()
    _lib().ref_philox4x32_10(c, k, o)
    return list(o)


def stochastic_round_e4m3fn(weight, scale=None, seed=0):
    """float.py:14-67 behind ops.py:419-426 (weight / scale_weight, float16, stochastic rounding to e4m3fn) with
    the uniform numbers of moe_ref.c (Philox, keyed by seed and element index). weight fp32 or bf16 -> e4m3fn."""
    is_bf16 = weight.dtype == torch.bfloat16
    src = weight.float().contiguous()
    out = torch.empty(weight.shape, dtype=torch.uint8)
    sc = None if scale is None else scale.detach().float().reshape(1).contiguous()
    _lib().ref_stochastic_round_e4m3fn(_p(src), src.numel(), None if sc is None else _p(sc), seed, int(is_bf16),
                                       _p(out))
    return out.view(torch.float8_e4m3fn)


# ------------------------------------------------------- feed-forward branch of a block

def ln_modulate_torch(x3, shift, scale, eps=1e-6):
    """model.py:430-431 / 516-517 with torch's own ops: x3 [B,S,D]; shift, scale [B,1,D], all one dtype."""
    n = F.layer_norm(x3, (x3.shape[-1],), None, None, eps).to(x3.dtype)
    return n * (1 + scale) + shift


def ln_modulate_c(x2d_bf16, shift_bf16, scale_bf16, tokens_per_batch, eps=1e-6):
    """The same in the fixed summation order of moe_ref.c ref_ln_modulate; x2d [T,D], shift/scale [B,D] bf16."""
    T, D = x2d_bf16.shape
    out = torch.empty((T, D), dtype=torch.bfloat16)
    rc = _lib().ref_ln_modulate(_p(x2d_bf16.contiguous()), _p(scale_bf16.contiguous()), _p(shift_bf16.contiguous()),
                                T, D, tokens_per_batch, eps, _p(out))
    if rc != 0:
        raise ValueError("ref_ln_modulate: bad shape")
    return out


def gated_residual_torch(y3, gate, residual3):
    """model.py:432-433 / 518-523: gate [B,1,D] * y [B,S,D] + residual."""
    return gate * y3 + residual3


def gated_residual_c(y2d_bf16, gate_bf16, residual2d_bf16, tokens_per_batch):
    T, D = y2d_bf16.shape
    out = torch.empty((T, D), dtype=torch.bfloat16)
    _lib().ref_gated_residual(_p(y2d_bf16.contiguous()), _p(gate_bf16.contiguous()), _p(residual2d_bf16.contiguous()),
                              ctypes.c_int(T), ctypes.c_int(D), ctypes.c_int(tokens_per_batch), _p(out))
    return out


def ff_branch(x3, shift, scale, gate, params, mode, gate_result=None, fixed_order_norm=False):
    """model.py:429-433: x + gate * ff(LayerNorm(x) * (1 + scale) + shift) for x3 [B,S,D], shift/scale/gate
    [B,1,D]. fixed_order_norm takes the LayerNorm statistics in ref_ln_modulate's order (what the HIP kernel
    does) instead of torch's. Returns (out, normed tokens)."""
    B, S, D = x3.shape
    if fixed_order_norm:
        n = ln_modulate_c(x3.reshape(-1, D), shift.reshape(B, D), scale.reshape(B, D), S).view(B, S, D)
    else:
        n = ln_modulate_torch(x3, shift, scale)
    y = moe_forward(n, params, mode, gate_result=gate_result)
    return gated_residual_torch(y, gate, x3), n


def moe_forward_dense(x, params, mode, topk_idx, topk_weight):
    """Brute force used to pin moe_forward: run EVERY expert on EVERY token and pick by mask.
    Same rounding points as moe_forward (slot products rounded, then summed)."""
    x2 = x.reshape(-1, x.shape[-1])
    outs = torch.stack([ffn_swiglu(x2, ffn, mode) for ffn in params["experts"]], dim=0)  # [E,T,D]
    T = x2.shape[0]
    sel = outs[topk_idx.long().t(), torch.arange(T).unsqueeze(0)]  # [K,T,D]
    y = (sel.permute(1, 0, 2) * topk_weight.to(x.dtype).unsqueeze(-1)).sum(dim=1)
    y = y.view(x.shape).to(x.dtype)
    return y + ffn_swiglu(x, params["shared"], mode)


def renorm_topk(topk_weight):
    """The optional renormalisation of MoEGate.forward (/root/reference/comfy/ldm/hidream/model.py:277-280) on the
    bf16 gate weights, as the three torch ops evaluate it: sum -> bf16, + 1e-20 -> bf16, quotient -> bf16."""
    denominator = topk_weight.sum(dim=-1, keepdim=True) + 1e-20
    return topk_weight / denominator


def error_metrics(got, ref):
    """rms(err)/rms(ref), max|err|/rms(ref), max|err|/max|ref| in fp64."""
    g = got.double().reshape(-1)
    r = ref.double().reshape(-1)
    err = (g - r).abs()
    rms_ref = float(r.pow(2).mean().sqrt())
    return {
        "rel_rms": float(err.pow(2).mean().sqrt()) / rms_ref,
        "max_over_rms": float(err.max()) / rms_ref,
        "max_over_max": float(err.max()) / float(r.abs().max()),
    }


def to_numpy_u16(t_bf16):
    return t_bf16.view(torch.int16).numpy().view(np.uint16)
