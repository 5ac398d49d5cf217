"""Hunyuan3D-2.1 mixture-of-experts block with the constructor and forward signatures, attribute names and
state-dict keys of the reference (/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:8-188), computing on
the MI355X with the same gate, dispatch and combine kernels as the HiDream layer and a grouped Linear with bias
and erf-GELU epilogue for the experts.

  GELU          hunyuandit.py:8-26    gelu(proj(x))
  FeedForward   hunyuandit.py:28-50   net = [GELU, Dropout, Linear]  (keys net.0.proj.*, net.2.*)
  MoEGate       hunyuandit.py:73-112  softmax scores, top-k of E unsorted, not renormalised
  MoEBlock      hunyuandit.py:114-188 experts on their tokens, weighted index_add_ in expert order, + shared expert

Inference only (the reference's training branch and auxiliary loss are not part of this path). A token meets at
most two experts, so the index_add_ accumulation bf16(bf16(w_a y_a) + bf16(w_b y_b)) is the same two-term sum the
HiDream combine forms. Inputs must be bf16 or fp16 HIP tensors (fp16 is what model_management.unet_dtype picks for
this model family on a device with fp16 support, supported_models_base.py:46): there is no CPU path. With fp16
every tensor and every rounding point of the block is fp16; scaled-fp8 Linears take bf16 activations only.

Two ways through the experts:
  * every Linear a plain one of the activation dtype resident on the device (no weight function, no scale_weight):
    two grouped launches for all experts and the shared expert;
  * anything else the `operations` argument brings (scaled-fp8 Linears with or without the fp8 matrix multiply,
    manual-cast or offloaded weights, weight functions): one expert at a time through the Linear modules' own
    forward, the GELU as an elementwise kernel, with the same gate, dispatch and combine kernels around them.
"""
import torch
import torch.nn as nn

from . import functional as HF
from . import ops as amd_ops

BF16 = torch.bfloat16
ACT_DTYPES = HF.ACT_DTYPES


class _LinearWithBias(amd_ops.disable_weight_init.Linear):
    """operations.Linear as the reference's default constructor makes it (bias=True); computes through the
    grouped kernel with a single group."""

    def forward(self, x):
        if not (x.is_cuda and x.dtype in ACT_DTYPES and self.weight.dtype == x.dtype):
            raise RuntimeError("comfyui_amd.hunyuan3d: expected bfloat16 or float16 HIP tensors and weights of the same "
                               "dtype; there is no CPU path")
        x2 = x.reshape(-1, x.shape[-1]).contiguous()
        _, y = HF.grouped_linear(x2[:0], None, [], a_static=x2, shared=(self.weight, self.bias), act="none")
        return y.view(*x.shape[:-1], self.weight.shape[0])


class _Operations:
    Linear = _LinearWithBias


class GELU(nn.Module):
    def __init__(self, dim_in: int, dim_out: int, operations, device, dtype):
        super().__init__()
        self.proj = operations.Linear(dim_in, dim_out, device=device, dtype=dtype)

    def forward(self, hidden_states):
        x2 = hidden_states.reshape(-1, hidden_states.shape[-1]).contiguous()
        _need(x2)
        if not _plain_bf16(self.proj, x2):
            return HF.gelu(self.proj(x2).contiguous()).view(*hidden_states.shape[:-1], self.proj.weight.shape[0])
        _, y = HF.grouped_linear(x2[:0], None, [], a_static=x2, shared=(self.proj.weight, self.proj.bias), act="gelu")
        return y.view(*hidden_states.shape[:-1], self.proj.weight.shape[0])


def _need(x):
    if not (x.is_cuda and x.dtype in ACT_DTYPES):
        raise RuntimeError(f"comfyui_amd.hunyuan3d: expected bfloat16 or float16 HIP activations, got {x.dtype} on "
                           f"{x.device}; there is no CPU path")


def _plain_bf16(lin, x):
    """True when `lin` can join a grouped launch as it stands: weight (and bias) of x's dtype (bf16 or fp16) on x's
    device, nothing to apply to them first."""
    if getattr(lin, "weight_function", None) or getattr(lin, "bias_function", None):
        return False
    if getattr(lin, "scale_weight", None) is not None:
        return False
    if lin.weight.dtype != x.dtype or lin.weight.device != x.device:
        return False
    return lin.bias is None or (lin.bias.dtype == x.dtype and lin.bias.device == x.device)


class FeedForward(nn.Module):
    def __init__(self, dim: int, dim_out=None, mult: int = 4, dropout: float = 0.0, inner_dim=None, operations=None,
                 device=None, dtype=None):
        super().__init__()
        operations = operations if operations is not None else _Operations
        if inner_dim is None:
            inner_dim = int(dim * mult)
        dim_out = dim_out if dim_out is not None else dim
        self.net = nn.ModuleList([])
        self.net.append(GELU(dim, inner_dim, operations=operations, device=device, dtype=dtype))
        self.net.append(nn.Dropout(dropout))
        self.net.append(operations.Linear(inner_dim, dim_out, device=device, dtype=dtype))

    def stage_weights(self):
        """((proj weight, bias), (out weight, bias))"""
        return (self.net[0].proj.weight, self.net[0].proj.bias), (self.net[2].weight, self.net[2].bias)

    def fusable(self, x):
        return _plain_bf16(self.net[0].proj, x) and _plain_bf16(self.net[2], x)

    def forward(self, hidden_states: torch.Tensor) -> torch.Tensor:
        x2 = hidden_states.reshape(-1, hidden_states.shape[-1]).contiguous()
        _need(x2)
        if not self.fusable(x2):
            y = self.net[2](self.net[0](x2))     # net[1] is Dropout, the identity at inference
            return y.view(*hidden_states.shape[:-1], y.shape[-1])
        w_in, w_out = self.stage_weights()
        _, h = HF.grouped_linear(x2[:0], None, [], a_static=x2, shared=w_in, act="gelu")
        _, y = HF.grouped_linear(h[:0], None, [], a_static=h, shared=w_out, act="none")
        return y.view(*hidden_states.shape[:-1], y.shape[-1])


class MoEGate(nn.Module):
    def __init__(self, embed_dim, num_experts=16, num_experts_per_tok=2, aux_loss_alpha=0.01, device=None, dtype=None):
        super().__init__()
        self.top_k = num_experts_per_tok
        self.n_routed_experts = num_experts
        self.alpha = aux_loss_alpha
        self.gating_dim = embed_dim
        self.weight = nn.Parameter(torch.empty((self.n_routed_experts, self.gating_dim), device=device, dtype=dtype))

    def forward(self, hidden_states: torch.Tensor):
        if self.top_k != 2:
            raise NotImplementedError("the HIP gate kernel selects the top 2 experts")
        x2 = hidden_states.reshape(-1, hidden_states.size(-1)).contiguous()
        gate_w = amd_ops.cast_to(self.weight, dtype=x2.dtype, device=x2.device).contiguous()
        idx, w = HF.gate_top2(x2, gate_w)
        return idx.to(torch.int64), w, None


class MoEBlock(nn.Module):
    def __init__(self, dim, num_experts: int = 6, moe_top_k: int = 2, dropout: float = 0.0, ff_inner_dim: int = None,
                 operations=None, device=None, dtype=None):
        super().__init__()
        self.moe_top_k = moe_top_k
        self.num_experts = num_experts
        self.experts = nn.ModuleList([
            FeedForward(dim, dropout=dropout, inner_dim=ff_inner_dim, operations=operations, device=device, dtype=dtype)
            for _ in range(num_experts)
        ])
        self.gate = MoEGate(dim, num_experts=num_experts, num_experts_per_tok=moe_top_k, device=device, dtype=dtype)
        self.shared_experts = FeedForward(dim, dropout=dropout, inner_dim=ff_inner_dim, operations=operations,
                                          device=device, dtype=dtype)

    def forward(self, hidden_states) -> torch.Tensor:
        if self.training:
            raise NotImplementedError("comfyui_amd.hunyuan3d.MoEBlock is inference only (call .eval())")
        if self.moe_top_k != 2:
            raise NotImplementedError("the HIP gate kernel selects the top 2 experts")
        orig_shape = hidden_states.shape
        x2 = hidden_states.reshape(-1, orig_shape[-1]).contiguous()
        _need(x2)
        gate_w = amd_ops.cast_to(self.gate.weight, dtype=x2.dtype, device=x2.device).contiguous()
        idx, w = HF.gate_top2(x2, gate_w)
        _, offsets, perm, inv_perm = HF.dispatch(idx, self.num_experts)
        if not (all(e.fusable(x2) for e in self.experts) and self.shared_experts.fusable(x2)):
            xs = HF.permute_bf16(x2, perm)
            y = torch.empty_like(xs)
            bounds = offsets.tolist()  # host sync: segment sizes steer the per-expert calls
            for i, expert in enumerate(self.experts):
                lo, hi = bounds[i], bounds[i + 1]
                if hi > lo:
                    y[lo:hi] = expert(xs[lo:hi])
            return HF.combine(y, inv_perm, w, self.shared_experts(x2)).view(*orig_shape)
        stage1 = [e.stage_weights()[0] for e in self.experts]
        stage2 = [e.stage_weights()[1] for e in self.experts]
        sh1, sh2 = self.shared_experts.stage_weights()
        # the experts' first Linear reads the routed rows through the permutation: no copy in expert order
        h, h_sh = HF.grouped_linear_tokens(x2, perm, offsets, stage1, shared=sh1, act="gelu")
        y, y_sh = HF.grouped_linear(h, offsets, stage2, a_static=h_sh, shared=sh2, act="none")
        return HF.combine(y, inv_perm, w, y_sh).view(*orig_shape)
