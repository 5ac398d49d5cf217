"""HiDream mixture-of-experts SwiGLU feed-forward modules with the constructor and
forward signatures, attribute names and state-dict keys of the reference
(/root/reference/comfy/ldm/hidream/model.py:215-325), computing on the MI355X.

  FeedForwardSwiGLU      model.py:215-238   w2(silu(w1 x) * w3 x)
  MoEGate                model.py:242-283   softmax scores, top-2 of E, not renormalised
  MOEFeedForwardSwiGLU   model.py:287-325   gate -> dispatch -> experts -> weighted sum -> + shared

State-dict keys per layer: shared_experts.{w1,w2,w3}.weight, experts.{i}.{w1,w2,w3}.weight,
gate.weight (+ .scale_weight / .scale_input under scaled-fp8 operations) -- the names LoRA
key maps and checkpoints address.

MOEFeedForwardSwiGLU.forward enqueues the whole layer through ONE library call when all
Linears share a supported storage dtype (bf16, or float8_e4m3fn with fp8 matrix multiply);
otherwise it composes the same HIP stages per expert through the Linear modules, which
needs the per-expert row counts on the host (one sync, as the reference's mask indexing).
Inputs must be bf16 HIP tensors: there is no CPU path.
"""
from typing import Optional

import torch
import torch.nn as nn

from . import functional as HF
from . import ops as amd_ops

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16


def _plain(lin):
    return (len(getattr(lin, "weight_function", ())) == 0 and len(getattr(lin, "bias_function", ())) == 0
            and lin.bias is None)


def _pack_ffn(ffn, x, wdt, keep):
    """hdmoe_ffn_weights for one FeedForwardSwiGLU whose Linears store `wdt`, or None when the three Linears
    cannot be served by the fused kernels (w1/w3 quantising the same input with different scale_input values).
    Tensors that must outlive the call are appended to `keep`."""
    fp8 = wdt == FP8
    dev = x.device
    scales = {}
    own = {}   # the Linear's own scale_input (Parameter or tensor, wherever it lives): the stable object to cache on
    ws = []
    for name, l in (("1", ffn.w1), ("2", ffn.w2), ("3", ffn.w3)):
        if _plain(l) and l.weight.device == dev:
            w = l.weight
        else:
            w, _ = amd_ops.cast_bias_weight(l, x, dtype=wdt)   # offloaded weights, weight functions (LowVramPatch)
        w = w.contiguous()
        keep.append(w)
        ws.append(w)
        if fp8:
            sw = getattr(l, "scale_weight", None)
            sw = amd_ops._one(dev) if sw is None else sw.to(dev)
            si = getattr(l, "scale_input", None)
            own[name] = si
            if si is not None:
                si = si.to(dev)
                keep.append(si)
            keep.append(sw)
            scales["scale_w" + name] = sw
            scales["scale_in" + name] = si
    same13 = False
    if fp8:
        s1, s3 = scales["scale_in1"], scales["scale_in3"]
        if (s1 is None) != (s3 is None):
            return None
        if s1 is not None and s1.data_ptr() != s3.data_ptr():
            # two tensors: the values are read from the Linears' own tensors (a host tensor of an offloaded module
            # costs no device synchronisation; a device Parameter is read once and cached)
            if amd_ops.scale_value(own["1"]) != amd_ops.scale_value(own["3"]):
                return None  # w1 and w3 quantise the same input differently: one fp8 copy cannot serve both
            same13 = True
    return HF.make_ffn_weights(ws[0], ws[1], ws[2], scales, same_scale_in13=same13)


def _fusable_dtype(ffns):
    """Common storage dtype of all Linears if the fused kernels can run them, else None."""
    lins = [l for f in ffns for l in (f.w1, f.w2, f.w3)]
    for l in lins:
        # any Linear that follows the operations contract (this package's or ComfyUI's own classes)
        if not isinstance(l, torch.nn.Linear) or l.bias is not None or len(getattr(l, "bias_function", ())) > 0:
            return None
    wdt = lins[0].weight.dtype
    if wdt not in (BF16, FP8) or any(l.weight.dtype != wdt for l in lins):
        return None
    if wdt == FP8 and not all(getattr(l, "hdmoe_fp8_matrix_mult", isinstance(l, amd_ops.fp8_ops.Linear)) for l in lins):
        return None  # scaled fp8 without fp8 matrix multiply: dequantising Linear path
    if wdt == FP8 and any(isinstance(l, amd_ops.fp8_ops.Linear) and l.training for l in lins):
        return None  # fp8_ops.Linear computes in the activation dtype while training (comfy/ops.py:368)
    return wdt


def _lin_tensors(l):
    """(weight, bias, scale_weight, scale_input) of a Linear, read from the module's own dictionaries: nn.Module's
    __getattr__ costs about as much per access as everything else here together."""
    d = l.__dict__
    p = d["_parameters"]
    sw = p["scale_weight"] if "scale_weight" in p else d.get("scale_weight")
    si = p["scale_input"] if "scale_input" in p else d.get("scale_input")
    return p["weight"], p.get("bias"), sw, si


def _pack_key(ffns, dev):
    """Everything the packed pointer structures of `ffns` depend on, or None when they cannot be reused from one call
    to the next (weights that are cast, moved or patched per call). Values of scale_input enter through the version
    counters and ops.invalidate_scale_cache(), as they do for ops.scale_value."""
    key = [dev, amd_ops._scale_epoch]
    for f in ffns:
        mods = f.__dict__["_modules"]
        for l in (mods["w1"], mods["w2"], mods["w3"]):
            w, b, sw, si = _lin_tensors(l)
            if w.device != dev or getattr(l, "weight_function", None) or getattr(l, "bias_function", None):
                return None
            if (sw is not None and sw.device != dev) or (si is not None and si.device != dev):
                return None
            # the cached structures hold raw addresses of the module's own tensors: a weight that has to be made
            # contiguous, or a scale that is not an fp32 scalar in place, is packed from a temporary every call
            if not w.is_contiguous() or any(t is not None and (t.dtype != torch.float32 or not t.is_contiguous())
                                            for t in (sw, si)):
                return None
            key.append((type(l), l.training, w.data_ptr(), w.dtype, b is None, getattr(l, "hdmoe_fp8_matrix_mult", None),
                        None if sw is None else (sw.data_ptr(), sw._version),
                        None if si is None else (si.data_ptr(), si._version)))
    return tuple(key)


def _gate_check(gate):
    """What the HIP gate kernel computes, checked on any gate module with the reference's attributes (this package's
    MoEGate or the reference's own, model.py:242-259)."""
    if getattr(gate, "scoring_func", "softmax") != 'softmax':
        raise NotImplementedError(f'insupportable scoring function for MoE gating: {gate.scoring_func}')
    if getattr(gate, "top_k", 2) != 2:
        raise NotImplementedError("the HIP gate kernel selects the top 2 experts")


def _gate_weight(gate, hidden_states):
    """The gate weight in the activations' dtype on their device (model.py:268 routes it through cast_to because a
    bare Parameter may have been left on the offload device)."""
    return amd_ops.cast_to(gate.weight, dtype=hidden_states.dtype, device=hidden_states.device).contiguous()


class FeedForwardSwiGLU(nn.Module):
    def __init__(self, dim: int, hidden_dim: int, multiple_of: int = 256,
                 ffn_dim_multiplier: Optional[float] = None, dtype=None, device=None, operations=None):
        super().__init__()
        hidden_dim = int(2 * hidden_dim / 3)
        if ffn_dim_multiplier is not None:
            hidden_dim = int(ffn_dim_multiplier * hidden_dim)
        hidden_dim = multiple_of * ((hidden_dim + multiple_of - 1) // multiple_of)
        operations = operations if operations is not None else amd_ops.disable_weight_init
        self.w1 = operations.Linear(dim, hidden_dim, bias=False, dtype=dtype, device=device)
        self.w2 = operations.Linear(hidden_dim, dim, bias=False, dtype=dtype, device=device)
        self.w3 = operations.Linear(dim, hidden_dim, bias=False, dtype=dtype, device=device)

    def forward(self, x):
        if x.is_cuda and x.dtype == BF16:
            wdt = _fusable_dtype([self])
            if wdt is not None:
                x2 = x.reshape(-1, x.shape[-1]).contiguous()
                keep = []
                packed = _pack_ffn(self, x2, wdt, keep)
                if packed is not None:
                    y = HF.ffn_swiglu(x2, packed, self.w1.weight.shape[0], wdt)
                    del keep
                    return y.view(*x.shape[:-1], self.w2.weight.shape[0])
        # per-Linear composition (also the place where a CPU tensor is refused)
        return self.w2(HF.silu_mul(self.w1(x), self.w3(x)))

    def forward_branch(self, x, shift, scale, gate, eps=1e-6):
        """The whole feed-forward branch of a block around a dense feed-forward (the text stream's `ff_t`, or `ff_i`
        of a block without routed experts; comfy/ldm/hidream/model.py:518-523, 402-403):
            x + gate * self(LayerNorm(x, eps, no affine) * (1 + scale) + shift)
        x [B,S,dim]; shift, scale, gate [B,1,dim] in bf16. Not a method of the reference class."""
        if x.dtype != BF16 or not x.is_cuda or x.dim() != 3:
            raise RuntimeError(f"FeedForwardSwiGLU.forward_branch: expected a [B,S,dim] bfloat16 HIP tensor, got "
                               f"{tuple(x.shape)} {x.dtype} on {x.device}; comfyui_amd has no CPU path")
        B, S, D = x.shape
        x2 = x.reshape(-1, D).contiguous()
        n = HF.ln_modulate(x2, scale.reshape(B, D).contiguous(), shift.reshape(B, D).contiguous(), S, eps)
        y = self.forward(n.view(B, S, D)).reshape(-1, D)
        return HF.gated_residual(y, gate.reshape(B, D).contiguous(), x2, S).view(B, S, D)


class MoEGate(nn.Module):
    def __init__(self, embed_dim, num_routed_experts=4, num_activated_experts=2, aux_loss_alpha=0.01,
                 dtype=None, device=None, operations=None):
        super().__init__()
        self.top_k = num_activated_experts
        self.n_routed_experts = num_routed_experts
        self.scoring_func = 'softmax'
        self.alpha = aux_loss_alpha
        self.seq_aux = False
        self.norm_topk_prob = False
        self.gating_dim = embed_dim
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, self.gating_dim), dtype=dtype, device=device))
        self.reset_parameters()

    def reset_parameters(self) -> None:
        pass

    def _check(self):
        _gate_check(self)

    def device_weight(self, hidden_states):
        return _gate_weight(self, hidden_states)

    def forward(self, hidden_states):
        self._check()
        bsz, seq_len, h = hidden_states.shape
        x2 = hidden_states.reshape(-1, h).contiguous()
        idx, w = HF.gate_top2(x2, self.device_weight(x2))
        if self.norm_topk_prob:   # model.py:277-280; HiDream leaves it off
            w = HF.renorm_top2(w)
        return idx.to(torch.int64), w, None


class MOEFeedForwardSwiGLU(nn.Module):
    def __init__(self, dim: int, hidden_dim: int, num_routed_experts: int, num_activated_experts: int,
                 dtype=None, device=None, operations=None):
        super().__init__()
        self.shared_experts = FeedForwardSwiGLU(dim, hidden_dim // 2, dtype=dtype, device=device, operations=operations)
        self.experts = nn.ModuleList([FeedForwardSwiGLU(dim, hidden_dim, dtype=dtype, device=device, operations=operations)
                                      for i in range(num_routed_experts)])
        self.gate = MoEGate(embed_dim=dim, num_routed_experts=num_routed_experts,
                            num_activated_experts=num_activated_experts, dtype=dtype, device=device,
                            operations=operations)
        self.num_activated_experts = num_activated_experts

    # Not an attribute of the reference class. Set `module.batch_invariant = True` to have every token's output bytes
    # independent of how the other tokens of the batch are routed: between a few hundred and about two thousand tokens
    # the down projection is cut along K and the cut that runs is otherwise picked from the experts' segment sizes,
    # which changes the fp32 summation order (the last bit of an output) with the rest of the batch.

    # ---- fused path ----------------------------------------------------------------

    def _collect(self, x):
        """Device pointers of all 15 Linears for the one-call path, or None when the layer
        needs the per-Linear composition. Returned tensors are kept alive by the caller."""
        ffns = list(self.experts) + [self.shared_experts]
        if amd_ops.take_scale_check(x.device):   # a kernel found a cached scale value stale: rebuild from the tensors
            self.__dict__["_packed"] = None
        # resident, unpatched weights: the structures of the previous call hold as long as nothing they were built
        # from has changed
        key = _pack_key(ffns, x.device)
        cached = self.__dict__.get("_packed")
        if key is not None and cached is not None and cached[0] == key:
            self.__dict__["_uniform_scale_in"] = cached[2]
            return cached[1]
        self.__dict__["_packed"] = None
        wdt = _fusable_dtype(ffns)
        if wdt is None:
            return None
        keep = []
        packed = []
        for f in ffns:
            fw = _pack_ffn(f, x, wdt, keep)
            if fw is None:
                return None
            packed.append(fw)
        # whether one scale_input value serves every Linear that reads the tokens (they are then cast to fp8 once) is
        # decided on the device from the values themselves; the attribute stays for callers of functional.moe_ffn
        uniform = False
        self.__dict__["_uniform_scale_in"] = uniform
        if key is not None:
            # the structures hold raw pointers of tensors the module owns and the key was read from: no tensor is
            # referenced from the cache (an offloaded or replaced weight must be free to go)
            self.__dict__["_packed"] = (key, (wdt, packed[:-1], packed[-1], ()), uniform)
        return wdt, packed[:-1], packed[-1], keep

    def forward(self, x, stage_events=None):
        """x [B,S,dim] -> [B,S,dim]. `stage_events` (optional, not in the reference signature) is a
        sequence of 7 hipEvent_t handles recorded around the six stages of the one-call path."""
        if x.dtype != BF16 or not x.is_cuda:
            raise RuntimeError(f"MOEFeedForwardSwiGLU: expected a bfloat16 HIP tensor, got {x.dtype} on {x.device}; "
                               "comfyui_amd has no CPU path")
        _gate_check(self.gate)      # any gate module with the reference's attributes, not only this package's
        orig_shape = x.shape
        x2 = x.reshape(-1, orig_shape[-1]).contiguous()
        gate_w = _gate_weight(self.gate, x2)
        # renormalised gate weights are not part of the one-call path: the stages are composed
        got = None if getattr(self.gate, "norm_topk_prob", False) else self._collect(x2)
        if got is not None:
            wdt, experts, shared, keep = got
            H = self.experts[0].w1.weight.shape[0]
            Hs = self.shared_experts.w1.weight.shape[0]
            y = HF.moe_ffn(x2, gate_w, experts, shared, H, Hs, wdt, stage_events=stage_events,
                           scale_check=amd_ops.scale_check_word(x2.device) if wdt == FP8 else None,
                           fixed_k_cut=self.__dict__.get("batch_invariant", False))
            del keep
            return y.view(*orig_shape)
        return self._forward_composed(x2, gate_w).view(*orig_shape)

    def forward_branch(self, x, shift, scale, gate, eps=1e-6, stage_events=None):
        """The whole feed-forward branch of a block in one enqueue (not a method of the reference class; it is
        the lines around its call, comfy/ldm/hidream/model.py:429-433 and 515-523):
            x + gate * self(LayerNorm(x, eps, no affine) * (1 + scale) + shift)
        x [B,S,dim]; shift, scale, gate [B,1,dim] (the chunks of adaLN_modulation) in bf16."""
        if x.dtype != BF16 or not x.is_cuda or x.dim() != 3:
            raise RuntimeError(f"MOEFeedForwardSwiGLU.forward_branch: expected a [B,S,dim] bfloat16 HIP tensor, got "
                               f"{tuple(x.shape)} {x.dtype} on {x.device}; comfyui_amd has no CPU path")
        _gate_check(self.gate)
        B, S, D = x.shape
        x2 = x.reshape(-1, D).contiguous()
        mods = tuple(m.reshape(B, D).contiguous() for m in (shift, scale, gate))
        gate_w = _gate_weight(self.gate, x2)
        got = None if getattr(self.gate, "norm_topk_prob", False) else self._collect(x2)
        if got is not None:
            wdt, experts, shared, keep = got
            H = self.experts[0].w1.weight.shape[0]
            Hs = self.shared_experts.w1.weight.shape[0]
            y = HF.moe_ffn(x2, gate_w, experts, shared, H, Hs, wdt, stage_events=stage_events, modulation=mods,
                           scale_check=amd_ops.scale_check_word(x2.device) if wdt == FP8 else None,
                           fixed_k_cut=self.__dict__.get("batch_invariant", False),
                           tokens_per_batch=S, ln_eps=eps)
            del keep
            return y.view(B, S, D)
        n = HF.ln_modulate(x2, mods[1], mods[0], S, eps)
        return self._forward_composed(n, gate_w, gated_residual=(mods[2], x2, S)).view(B, S, D)

    # ---- composed path -----------------------------------------------------------------

    def _forward_composed(self, x2, gate_w, gated_residual=None):
        """Same stages, one expert at a time through the Linear modules (weight functions,
        offloaded or mixed-dtype weights, dequantising scaled-fp8 Linears)."""
        E = len(self.experts)
        idx, w = HF.gate_top2(x2, gate_w)
        if getattr(self.gate, "norm_topk_prob", False):
            w = HF.renorm_top2(w)
        counts, offsets, perm, inv_perm = HF.dispatch(idx, E)
        xs = HF.permute_bf16(x2, perm)
        y = torch.empty_like(xs)
        bounds = offsets.tolist()  # host sync: segment sizes steer the per-expert calls
        for i, expert in enumerate(self.experts):
            lo, hi = bounds[i], bounds[i + 1]
            if hi > lo:
                y[lo:hi] = expert(xs[lo:hi])
        shared = self.shared_experts(x2)
        if gated_residual is not None:
            g, res, per_batch = gated_residual
            return HF.combine_gated_residual(y, inv_perm, w, shared, g, res, per_batch)
        return HF.combine(y, inv_perm, w, shared)
