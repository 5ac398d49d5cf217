"""Host-side contract of the operation classes and modules: what ModelPatcher, LoRA patching and offload rely on
(/root/reference/comfy/ops.py:97-115, 282-284, 379-428, 449-473; comfy/model_patcher.py:98-107, 151-173;
comfy/ldm/hidream/model.py:215-325). Runs without a GPU; compute calls must refuse CPU tensors."""
import os
import re

import pytest
import torch

from comfyui_amd import hidream, ops, synth
from comfyui_amd.float_round import stochastic_rounding

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

EXPECTED_KEYS = (["shared_experts.w1.weight", "shared_experts.w2.weight", "shared_experts.w3.weight"]
                 + [f"experts.{e}.{w}.weight" for e in range(4) for w in ("w1", "w2", "w3")] + ["gate.weight"])


def test_state_dict_keys_and_shapes_match_reference_layout():
    m = hidream.MOEFeedForwardSwiGLU(2560, 4 * 2560, 4, 2, dtype=BF16, device="meta", operations=ops.disable_weight_init)
    assert list(m.state_dict().keys()) == EXPECTED_KEYS
    assert m.experts[0].w1.weight.shape == (6912, 2560) and m.experts[0].w2.weight.shape == (2560, 6912)
    assert m.shared_experts.w1.weight.shape == (3584, 2560) and m.gate.weight.shape == (4, 2560)
    assert m.experts[0].w1.bias is None and m.num_activated_experts == 2
    assert not hasattr(m.gate, "comfy_cast_weights")          # bare Parameter: never low-vram'd (model.py:255)
    assert m.gate.top_k == 2 and m.gate.n_routed_experts == 4 and m.gate.norm_topk_prob is False


def test_scaled_fp8_module_keys_and_parameters():
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=True, override_dtype=FP8)
    m = hidream.MOEFeedForwardSwiGLU(256, 1024, 4, 2, dtype=BF16, device="cpu", operations=cls)
    keys = list(m.state_dict().keys())
    assert keys[:3] == ["shared_experts.w1.weight", "shared_experts.w1.scale_weight", "shared_experts.w1.scale_input"]
    lin = m.experts[2].w3
    assert lin.weight.dtype == FP8 and lin.scale_weight.dtype == torch.float32 and lin.scale_weight.shape == ()
    assert isinstance(lin.scale_input, torch.nn.Parameter) and not lin.scale_weight.requires_grad
    assert m.gate.weight.dtype == BF16                         # the gate stays in the model dtype
    cls2 = ops.scaled_fp8_ops(fp8_matrix_mult=False, scale_input=False, override_dtype=FP8)
    lin2 = cls2.Linear(64, 128, bias=False, dtype=BF16)
    assert lin2.scale_input is None and "scale_input" not in lin2.state_dict() and lin2.weight.dtype == FP8


def test_cast_weight_bias_op_attributes_and_dispatch():
    for cls, cast in ((ops.disable_weight_init, False), (ops.manual_cast, True), (ops.fp8_ops, True)):
        lin = cls.Linear(64, 256, bias=False, dtype=BF16)
        assert lin.comfy_cast_weights is cast and lin.weight_function == [] and lin.bias_function == []
        assert isinstance(lin, torch.nn.Linear) and isinstance(lin, ops.CastWeightBiasOp)
    lin = ops.fp8_ops.Linear(64, 256, bias=False, dtype=FP8)
    assert lin.scale_weight is None and lin.scale_input is None
    # the per-instance flags ModelPatcher toggles (model_patcher.py:98-107, 694-722)
    lin = ops.disable_weight_init.Linear(64, 256, bias=False, dtype=BF16)
    called = []
    lin.forward_comfy_cast_weights = lambda x: called.append("cast") or x
    lin.prev_comfy_cast_weights = lin.comfy_cast_weights
    lin.comfy_cast_weights = True
    lin(torch.zeros(1, 64, dtype=BF16))
    lin.comfy_cast_weights = False
    lin.weight_function = [lambda w: w]
    lin(torch.zeros(1, 64, dtype=BF16))
    assert called == ["cast", "cast"]


def test_cast_to_and_cast_bias_weight_semantics():
    w = torch.randn(8, 8)
    assert ops.cast_to(w) is w and ops.cast_to(w, torch.float32, w.device) is w
    c = ops.cast_to(w, torch.float32, w.device, copy=True)
    assert c is not w and torch.equal(c, w)
    assert ops.cast_to(w, BF16).dtype == BF16
    lin = ops.manual_cast.Linear(8, 8, bias=False, dtype=torch.float32)
    with torch.no_grad():
        lin.weight.copy_(w)
    x = torch.zeros(2, 8, dtype=BF16)
    weight, bias = ops.cast_bias_weight(lin, x)
    assert weight.dtype == BF16 and bias is None
    lin.weight_function = [lambda t: t * 2]
    weight2, _ = ops.cast_bias_weight(lin, x)
    assert torch.equal(weight2, (w.to(BF16) * 2)) and torch.equal(lin.weight, w)      # functions act on a copy


def test_pick_operations_policy_without_fp8_compute():
    assert ops.supports_fp8_compute() is False                 # no gfx950 device in this process
    cls = ops.pick_operations(FP8, BF16, scaled_fp8=FP8, fp8_optimizations=True)
    lin = cls.Linear(64, 128, bias=False)
    assert lin.weight.dtype == FP8 and lin.hdmoe_fp8_matrix_mult is False and lin.scale_input is not None
    assert ops.pick_operations(BF16, BF16) is ops.disable_weight_init
    assert ops.pick_operations(BF16, None) is ops.disable_weight_init
    assert ops.pick_operations(torch.float16, BF16) is ops.manual_cast
    assert ops.pick_operations(FP8, BF16, fp8_optimizations=True) is ops.manual_cast   # fp8 compute unavailable


def test_convert_and_set_weight_round_trip():
    cls = ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=True, override_dtype=FP8)
    lin = cls.Linear(64, 128, bias=False, dtype=BF16)
    g = torch.Generator().manual_seed(0)
    w = torch.randn((128, 64), generator=g) * 0.02
    w8, s = synth.quantize_per_tensor(w)
    lin.weight = torch.nn.Parameter(w8, requires_grad=False)
    with torch.no_grad():
        lin.scale_weight.copy_(s)
    real = lin.convert_weight(lin.weight.to(torch.float32))
    assert torch.allclose(real, w8.float() * s)
    # exactly representable values come back unchanged except where the float16 noise add rounds up to the next
    # step (a property of the algorithm: the noise is added in float16), which is rare and only ever one step out
    back = lin.set_weight(real, seed=123, return_weight=True)
    assert back.dtype == FP8
    same = back.float() == w8.float()
    assert float(same.float().mean()) > 0.99
    ratio = (back.float()[~same] / w8.float()[~same])
    assert bool(((ratio > 1.0) & (ratio <= 1.126)).all())
    old = lin.weight
    lin.set_weight(real * 1.0, seed=1)
    assert lin.weight is not old and isinstance(lin.weight, torch.nn.Parameter) and lin.weight.dtype == FP8
    lin.set_weight(real, inplace_update=True, seed=1)
    # both hooks are found by name the way model_patcher.get_key_weight looks them up
    assert callable(getattr(lin, "set_weight")) and callable(getattr(lin, "convert_weight"))


def test_stochastic_rounding_is_unbiased_and_lands_on_neighbours():
    x = torch.full((4096, 16), 0.3)                    # between the e4m3 neighbours 0.28125 and 0.3125
    r = stochastic_rounding(x, FP8, seed=0).float()
    assert set(r.unique().tolist()) == {0.28125, 0.3125}
    assert abs(float(r.mean()) - 0.3) < 5e-4
    assert torch.equal(stochastic_rounding(x, FP8, seed=7), stochastic_rounding(x, FP8, seed=7))
    big = torch.tensor([[1000.0, -1000.0, 0.0, 448.0]])
    assert stochastic_rounding(big, FP8, seed=0).float().tolist() == [[448.0, -448.0, 0.0, 448.0]]
    assert stochastic_rounding(x, BF16).dtype == BF16


def test_cpu_tensors_are_refused_not_computed():
    sd, _ = synth.make_weights(0, dim=256)
    m = synth.build_module(synth.to_state_dict(sd, "fp8"), "fp8", "cpu", dim=256)
    x = torch.zeros(1, 4, 256, dtype=BF16)
    with pytest.raises(RuntimeError, match="no CPU path"):
        m(x)
    with pytest.raises(RuntimeError, match="no CPU path"):
        m.gate(x)
    with pytest.raises(RuntimeError, match="no CPU path"):
        m.experts[0](x)
    with pytest.raises(RuntimeError):
        m(x.float())


def test_product_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "comfyui_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M), f
                assert "libhdmoe_oracle" not in text and "moe_ref" not in text, f


def test_scale_cache_is_not_fooled_by_a_reused_id_or_address():
    """The host copy of a device scale is cached per parameter object; an entry left by a freed tensor whose id and
    address a new tensor happens to reuse must not be served for the new one. (Host tensors are read directly; the
    cache is exercised here on host tensors by asking for it.)"""
    import weakref
    from comfyui_amd import ops
    old = torch.nn.Parameter(torch.tensor(3.0), requires_grad=False)
    new = torch.nn.Parameter(torch.tensor(0.25), requires_grad=False)
    ops._scale_cache[id(new)] = (weakref.ref(old), new._version, new.data_ptr(), 3.0, ops._scale_epoch)
    assert ops.scale_value(new, use_cache=True) == 0.25
    assert ops.scale_value(new, use_cache=True) == 0.25          # now served from the refreshed entry
    with torch.no_grad():
        new.fill_(0.5)                                 # in-place update bumps the version
    assert ops.scale_value(new, use_cache=True) == 0.5


def test_scale_cache_is_dropped_on_load_and_on_request():
    """`p.data.copy_()`, which is how a state dict is loaded and how ModelPatcher writes in place, does not bump the
    version counter: the cache is dropped whenever a Linear of this package loads a state dict, and on request."""
    from comfyui_amd import ops
    p = torch.nn.Parameter(torch.tensor(2.0), requires_grad=False)
    assert ops.scale_value(p, use_cache=True) == 2.0
    p.data.copy_(torch.tensor(4.0))
    assert ops.scale_value(p, use_cache=True) == 2.0             # the stale entry the hooks exist for
    ops.invalidate_scale_cache()
    assert ops.scale_value(p, use_cache=True) == 4.0
    p.data.copy_(torch.tensor(8.0))
    lin = ops.disable_weight_init.Linear(4, 4, bias=False)
    lin.load_state_dict({"weight": torch.zeros(4, 4)})
    assert ops.scale_value(p, use_cache=True) == 8.0
    assert ops.scale_value(p) == 8.0                             # host tensors are read directly by default


def test_pointer_cache_refuses_tensors_that_would_be_packed_from_a_temporary():
    """The cached pointer structures hold raw addresses of the module's own tensors. A weight that is not contiguous
    is packed from a `contiguous()` temporary, and a scale that is not an fp32 scalar from a cast copy: neither may be
    cached, or the next call would read memory the allocator has taken back."""
    dev = torch.device("cpu")
    ffn = hidream.FeedForwardSwiGLU(64, 96, multiple_of=64, dtype=BF16, operations=ops.disable_weight_init)
    assert hidream._pack_key([ffn], dev) is not None
    w = ffn.w1.weight
    ffn.w1.weight = torch.nn.Parameter(torch.empty((w.shape[1], w.shape[0]), dtype=BF16).t(), requires_grad=False)
    assert ffn.w1.weight.shape == w.shape and not ffn.w1.weight.is_contiguous()
    assert hidream._pack_key([ffn], dev) is None
    ffn.w1.weight = w
    assert hidream._pack_key([ffn], dev) is not None
    ffn.w2.scale_input = torch.nn.Parameter(torch.ones((), dtype=torch.float64), requires_grad=False)
    assert hidream._pack_key([ffn], dev) is None
    ffn.w2.scale_input = torch.nn.Parameter(torch.ones(2, dtype=torch.float32)[::2].reshape(()), requires_grad=False)
    assert hidream._pack_key([ffn], dev) is not None      # a 0-dim view is contiguous: its address is its value's


def test_fp8_ops_linear_falls_back_when_the_fp8_path_raises(monkeypatch, caplog):
    """comfy/ops.py:367-377: an exception inside fp8_linear is logged and the Linear is computed the plain way."""
    import logging
    from comfyui_amd import ops
    lin = ops.fp8_ops.Linear(8, 8, bias=False, dtype=torch.float8_e4m3fn).eval()
    calls = []
    monkeypatch.setattr(ops, "fp8_linear", lambda self, x: (_ for _ in ()).throw(TypeError("no fp8 for this input")))
    monkeypatch.setattr(ops, "_linear_bf16", lambda x, w, b: calls.append((x.dtype, w.dtype)) or "plain result")
    with caplog.at_level(logging.INFO):
        out = lin.forward_comfy_cast_weights(torch.zeros((2, 8), dtype=torch.bfloat16))
    assert out == "plain result" and calls == [(torch.bfloat16, torch.bfloat16)]
    assert any("Exception during fp8 op" in r.message for r in caplog.records)
