"""The module swap of a loaded model the way a custom node does it: this package's MOEFeedForwardSwiGLU is assembled
around sub-modules that stay the HOST FRAMEWORK's own classes (its Linear, its feed-forward container, its gate), as
`ModelPatcher.add_object_patch` leaves them (/root/reference/comfy/model_patcher.py:453, 746-749). The classes
below are written for this test from the operations contract alone (/root/reference/comfy/ops.py:97-100: the
attributes `comfy_cast_weights`, `weight_function`, `bias_function`; :388-397: `scale_weight` / `scale_input`
Parameters; comfy/ldm/hidream/model.py:215-259: the attribute names w1/w2/w3, shared_experts, experts, gate and the
gate's fields): none of them derives from a class of this package, and their own forward raises, so whatever
output appears came through the one-call path.

Covered: the one-call path is taken and agrees with the oracle; a weight function appended at run time (LowVramPatch
style, model_patcher.py:594-619) is honoured; a Parameter replaced or written in place (comfy/utils.py:743-752) is
picked up; scale_input tensors written in place with `.data.copy_()` (no version bump, no call into this package)
give the right output, for all Linears at once and for one expert alone; w1 and w3 of one feed-forward drifting
apart the same way is caught on the device (NaN out and a raised check word, never a wrong number) and the next
forward runs the composed path."""
import pytest
import torch

from comfyui_amd import hidream, ops, synth
from oracle import hidream_moe_oracle as O
from tests.helpers import oracle_params, small_layer
from tests.test_gpu_layer import check_layer

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
FP8 = torch.float8_e4m3fn


class HostLinear(torch.nn.Linear):
    """A scaled-fp8 Linear as the host framework owns it, seen from outside."""
    comfy_cast_weights = True
    weight_function = []
    bias_function = []
    hdmoe_fp8_matrix_mult = True      # what the integrator sets: "this Linear runs fp8_linear"

    def __init__(self, in_features, out_features, device=None):
        super().__init__(in_features, out_features, bias=False, device=device, dtype=FP8)
        self.scale_weight = torch.nn.Parameter(torch.ones((), device=device, dtype=torch.float32), requires_grad=False)
        self.scale_input = torch.nn.Parameter(torch.ones((), device=device, dtype=torch.float32), requires_grad=False)

    def reset_parameters(self):
        return None

    def forward(self, x):
        raise AssertionError("the host framework's own Linear.forward must not run on the one-call path")


class HostFeedForward(torch.nn.Module):
    def __init__(self, dim, hidden, device):
        super().__init__()
        self.w1, self.w2, self.w3 = HostLinear(dim, hidden, device), HostLinear(hidden, dim, device), HostLinear(dim, hidden, device)

    def forward(self, x):
        raise AssertionError("the host framework's own feed-forward must not run on the one-call path")


class HostGate(torch.nn.Module):
    def __init__(self, dim, experts, device):
        super().__init__()
        self.top_k, self.n_routed_experts, self.scoring_func = 2, experts, 'softmax'
        self.alpha, self.seq_aux, self.norm_topk_prob, self.gating_dim = 0.01, False, False, dim
        self.weight = torch.nn.Parameter(torch.empty((experts, dim), dtype=BF16, device=device))


class HostMoE(torch.nn.Module):
    def __init__(self, dim, hidden, hidden_shared, experts, device):
        super().__init__()
        self.shared_experts = HostFeedForward(dim, hidden_shared, device)
        self.experts = torch.nn.ModuleList([HostFeedForward(dim, hidden, device) for _ in range(experts)])
        self.gate = HostGate(dim, experts, device)
        self.num_activated_experts = 2


def to_amd(ff):
    """The recipe a custom node uses: a module of this package around the host's own sub-modules."""
    new = hidream.MOEFeedForwardSwiGLU.__new__(hidream.MOEFeedForwardSwiGLU)
    torch.nn.Module.__init__(new)
    new.shared_experts, new.experts, new.gate = ff.shared_experts, ff.experts, ff.gate
    new.num_activated_experts = ff.num_activated_experts
    return new


def build(dev, seed=31, dim=512, tokens=600):
    sd, x = small_layer(seed=seed, dim=dim, tokens=tokens, weights="fp8", batch=2)
    H, Hs = sd["experts.0.w1.weight"].shape[0], sd["shared_experts.w1.weight"].shape[0]
    host = HostMoE(dim, H, Hs, 4, dev)
    host.load_state_dict({k: v.to(dev) for k, v in sd.items()})
    return sd, x, host.eval(), to_amd(host).eval()


def run(m, x, dev):
    from comfyui_amd import functional as HF
    xd = x.to(dev)
    with torch.no_grad():
        y = m(xd)
        idx, w = HF.gate_top2(xd.reshape(-1, x.shape[-1]), m.gate.weight)
    torch.cuda.synchronize()
    return y.cpu(), idx.cpu(), w.cpu()


def test_host_framework_linears_take_the_one_call_path(dev, monkeypatch):
    from comfyui_amd import functional as HF
    sd, x, host, m = build(dev)
    assert not any(isinstance(l, ops.disable_weight_init.Linear) for l in m.modules())
    calls = []
    real = HF.moe_ffn
    monkeypatch.setattr(HF, "moe_ffn", lambda *a, **k: calls.append(1) or real(*a, **k))
    y, idx, w = run(m, x, dev)
    assert calls == [1] and y.shape == x.shape
    check_layer(sd, x, "fp8", y, idx, w, 4)
    # the block's branch form goes the same way
    g = torch.Generator().manual_seed(3)
    B, S, D = x.shape
    shift, scale, gate = ((torch.randn((B, 1, D), generator=g) * 0.2).to(BF16) for _ in range(3))
    out = m.forward_branch(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    n = O.ln_modulate_c(x.reshape(-1, D), shift.reshape(B, D), scale.reshape(B, D), S).view(B, S, D)
    i2, w2, _, _ = O.gate_fixed_order(n.reshape(-1, D), sd["gate.weight"])
    ref = gate * O.moe_forward(n, oracle_params(sd, 4), "fp8mm", gate_result=(i2, w2)) + x
    met = O.error_metrics(out, ref)
    assert calls == [1, 1] and met["rel_rms"] <= 1e-2 and met["max_over_max"] <= 3e-2, met


def test_weight_function_appended_at_run_time(dev):
    """A low-VRAM patch object lands in `weight_function` of one Linear between two forwards (an instance attribute
    shadowing the class's empty list): the next forward multiplies with the patched weight."""
    sd, x, host, m = build(dev, seed=32)
    run(m, x, dev)                                    # fills the pointer cache with the unpatched weights
    halve = lambda w: (w.float() * 0.5).to(w.dtype)   # exact on e4m3 except in the subnormal range; the oracle does the same
    host.experts[1].w3.weight_function = [halve]
    sd2 = dict(sd)
    sd2["experts.1.w3.weight"] = halve(sd["experts.1.w3.weight"])
    y, idx, w = run(m, x, dev)
    check_layer(sd2, x, "fp8", y, idx, w, 4)
    host.experts[1].w3.weight_function = []
    y0, idx, w = run(m, x, dev)
    check_layer(sd, x, "fp8", y0, idx, w, 4)
    assert not torch.equal(y, y0)


def test_replaced_and_rewritten_parameters(dev):
    """ModelPatcher puts patched weights back either as a new Parameter object or by copying into the old one
    (/root/reference/comfy/utils.py:743-752); both must show in the next forward."""
    sd, x, host, m = build(dev, seed=33)
    run(m, x, dev)
    g = torch.Generator().manual_seed(5)
    w_new, s_new = synth.quantize_per_tensor(torch.randn(sd["experts.2.w2.weight"].shape, generator=g) * 0.03)
    sd2 = dict(sd)
    sd2["experts.2.w2.weight"], sd2["experts.2.w2.scale_weight"] = w_new, s_new.float().reshape(())
    host.experts[2].w2.weight = torch.nn.Parameter(w_new.to(dev), requires_grad=False)      # a new object
    host.experts[2].w2.scale_weight.data.copy_(s_new.float().reshape(()))                  # in place, no version bump
    y, idx, w = run(m, x, dev)
    check_layer(sd2, x, "fp8", y, idx, w, 4)
    w_new3, _ = synth.quantize_per_tensor(torch.randn(sd["shared_experts.w1.weight"].shape, generator=g) * 0.03)
    sd2["shared_experts.w1.weight"] = w_new3
    host.shared_experts.w1.weight.data.copy_(w_new3.to(dev))                                # in place
    y, idx, w = run(m, x, dev)
    check_layer(sd2, x, "fp8", y, idx, w, 4)


@pytest.mark.parametrize("dim,tokens", [(512, 600), (2560, 700)])   # the second: the sizes the 4-wave gate/up kernel takes
def test_scale_input_written_in_place(dev, dim, tokens):
    """`p.data.copy_()` on scale_input tensors between forwards, nothing of this package called: first every Linear
    gets the same new value (the tokens are still cast once), then one expert alone (the kernels go over to a cast per
    slot by themselves). Values that are not powers of two, so only the oracle of the same dataflow is gated."""
    sd, x, host, m = build(dev, seed=34, dim=dim, tokens=tokens)
    run(m, x, dev)
    sd2 = dict(sd)
    for name, lin in host.named_modules():
        if isinstance(lin, HostLinear):
            v = torch.tensor(0.37 if name.endswith(("w1", "w3")) else 0.21)
            lin.scale_input.data.copy_(v)
            sd2[name + ".scale_input"] = v
    y, idx, w = run(m, x, dev)
    check_layer(sd2, x, "fp8", y, idx, w, 4, gate_f32=False)
    for lin_name in ("w1", "w3"):
        v = torch.tensor(0.55)
        getattr(host.experts[3], lin_name).scale_input.data.copy_(v)
        sd2[f"experts.3.{lin_name}.scale_input"] = v
    y2, idx, w = run(m, x, dev)
    check_layer(sd2, x, "fp8", y2, idx, w, 4, gate_f32=False)
    assert not torch.equal(y, y2)
    assert int(ops.scale_check_word(dev)[0]) == 0


def test_w1_and_w3_drifting_apart_in_place_is_caught_on_the_device(dev):
    """The one decision the host takes from scale VALUES is whether w1 and w3 of a feed-forward share their cast (if
    not, the layer is composed per Linear). A stale answer cannot be noticed on the host without reading the device;
    the casting kernel compares the two factors itself: that forward returns NaN, the check word is raised, and the
    next forward, having dropped the cached values, is right again (through the composed path, i.e. the host
    framework's own Linear.forward, stood in for here by this package's fp8_linear)."""
    sd, x, host, m = build(dev, seed=35)
    run(m, x, dev)
    v = torch.tensor(0.6)
    host.experts[0].w3.scale_input.data.copy_(v)
    sd2 = dict(sd)
    sd2["experts.0.w3.scale_input"] = v
    y, idx, w = run(m, x, dev)
    assert bool(torch.isnan(y.float()).any()), "a cast made with the wrong factor must not pass as a number"
    assert int(ops.scale_check_word(dev)[0]) == 1
    for mod in list(host.modules()):                  # the composed path calls the host's own forwards
        if isinstance(mod, HostLinear):
            mod.forward = (lambda lin: lambda inp: ops.fp8_linear(lin, inp))(mod)
        elif isinstance(mod, HostFeedForward):
            mod.forward = (lambda f: lambda inp: f.w2(__import__("comfyui_amd").functional.silu_mul(f.w1(inp), f.w3(inp))))(mod)
    y, idx, w = run(m, x, dev)
    assert int(ops.scale_check_word(dev)[0]) == 0
    check_layer(sd2, x, "fp8", y, idx, w, 4, gate_f32=False)
