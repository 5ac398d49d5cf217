"""Scaled-fp8 checkpoint ingestion (/root/reference/comfy/model_detection.py:693-702, comfy/model_base.py:326-327,
comfy/utils.py:53-66): marker rules, layer discovery from the key set, module construction and loading."""
import os

import pytest
import torch
from safetensors.torch import save_file

from comfyui_amd import checkpoint as C
from comfyui_amd import ops as amd_ops
from comfyui_amd import synth

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16
PRE = "model.diffusion_model."


def model_state_dict(weights, layers=("double_stream_blocks.0.block.ff_i", "single_stream_blocks.5.block.ff_i"),
                     dim=256, hidden_arg=1024, experts=4, seed=3):
    full = {}
    for i, name in enumerate(layers):
        master, _ = synth.make_weights(seed + i, dim=dim, hidden_arg=hidden_arg, num_experts=experts)
        for k, v in synth.to_state_dict(master, weights).items():
            full[f"{PRE}{name}.{k}"] = v
    full[PRE + "x_embedder.proj.weight"] = torch.zeros(4, 4)     # something that is not a feed-forward
    return full


def test_marker_rules():
    # dtype of the marker = storage dtype; float32 stands for e4m3fn; two elements switch the optimisations off
    sd = {PRE + "scaled_fp8": torch.zeros(0, dtype=FP8)}
    assert C.read_scaled_fp8_marker(sd, PRE) == (FP8, True) and sd == {}
    assert C.read_scaled_fp8_marker({PRE + "scaled_fp8": torch.zeros(2, dtype=FP8)}, PRE) == (FP8, False)
    assert C.read_scaled_fp8_marker({PRE + "scaled_fp8": torch.zeros(1, dtype=torch.float32)}, PRE) == (FP8, True)
    assert C.read_scaled_fp8_marker({PRE + "scaled_fp8": torch.zeros(0, dtype=torch.float8_e5m2)}, PRE) == (torch.float8_e5m2, True)
    assert C.read_scaled_fp8_marker({"other": torch.zeros(1)}, PRE) == (None, False)
    assert C.scaled_fp8_marker(FP8, True).nelement() == 0 and C.scaled_fp8_marker(FP8, False).nelement() == 2
    assert C.scaled_fp8_marker(FP8).dtype == FP8


def test_layers_are_found_from_the_key_set():
    sd = model_state_dict("fp8")
    found = C.find_moe_layers(sd, PRE)
    assert sorted(found) == [PRE + "double_stream_blocks.0.block.ff_i", PRE + "single_stream_blocks.5.block.ff_i"]
    hs, hr = synth.swiglu_hidden(512), synth.swiglu_hidden(1024)
    for shp in found.values():
        assert shp == dict(dim=256, experts=4, hidden=hr, hidden_shared=hs)
    # a gate without its experts is not a layer; an incomplete expert list is an error
    assert C.find_moe_layers({"a.gate.weight": (4, 256)}) == {}
    broken = {k: v for k, v in sd.items() if ".experts.3.w2." not in k}
    with pytest.raises(KeyError):
        C.find_moe_layers(broken, PRE)
    assert C.find_moe_layers(sd, "some.other.prefix.") == {}


@pytest.mark.parametrize("optimizations", [True, False])
def test_scaled_fp8_file_builds_the_right_modules(tmp_path, optimizations):
    sd = model_state_dict("fp8")
    if not optimizations:
        sd = {k: v for k, v in sd.items() if not k.endswith("scale_input")}
    sd[PRE + "scaled_fp8"] = C.scaled_fp8_marker(FP8, optimizations)
    path = os.path.join(tmp_path, "model.safetensors")
    save_file(sd, path)
    modules, info = C.load_moe_layers(path, prefix=PRE)
    assert info["scaled_fp8"] == FP8 and info["fp8_optimizations"] is optimizations
    assert len(modules) == 2
    for layer, m in modules.items():
        assert type(m).__name__ == "MOEFeedForwardSwiGLU" and len(m.experts) == 4
        for ffn in list(m.experts) + [m.shared_experts]:
            for name in ("w1", "w2", "w3"):
                lin = getattr(ffn, name)
                key = f"{layer}.{'shared_experts' if ffn is m.shared_experts else 'experts.' + str(list(m.experts).index(ffn))}.{name}"
                assert lin.weight.dtype == FP8
                assert torch.equal(lin.weight.data.view(torch.uint8), sd[key + ".weight"].view(torch.uint8))
                assert torch.equal(lin.scale_weight.data, sd[key + ".scale_weight"])
                # scale_input exists exactly when the marker enables the optimisations (ops.py:388-397)
                assert (lin.scale_input is not None) is optimizations
                assert lin.bias is None
        assert m.gate.weight.dtype == BF16 and torch.equal(m.gate.weight.data, sd[layer + ".gate.weight"])
    # without a GPU there is no fp8 matrix multiply, whatever the marker says (ops.py:449-452)
    lin = next(iter(modules.values())).experts[0].w1
    assert lin.hdmoe_fp8_matrix_mult is False


def test_bf16_file_and_state_dict_source(tmp_path):
    sd = model_state_dict("bf16", layers=("double_stream_blocks.1.block.ff_i",))
    modules, info = C.load_moe_layers(sd, prefix=PRE)                  # a state dict instead of a path
    assert info["scaled_fp8"] is None and info["operations"] is amd_ops.disable_weight_init
    (layer, m), = modules.items()
    assert m.experts[2].w3.weight.dtype == BF16
    assert torch.equal(m.experts[2].w3.weight.data, sd[layer + ".experts.2.w3.weight"])
    assert PRE + "x_embedder.proj.weight" in sd                        # the caller's dict is left alone
    # only one of the layers on request
    sd2 = model_state_dict("bf16")
    want = PRE + "single_stream_blocks.5.block.ff_i"
    modules, _ = C.load_moe_layers(sd2, prefix=PRE, layers=[want])
    assert list(modules) == [want]


def test_errors_name_the_key(tmp_path):
    sd = model_state_dict("fp8", layers=("double_stream_blocks.0.block.ff_i",))
    sd[PRE + "scaled_fp8"] = C.scaled_fp8_marker(FP8)
    layer = PRE + "double_stream_blocks.0.block.ff_i"
    bad = dict(sd)
    del bad[layer + ".experts.1.w2.scale_weight"]
    with pytest.raises(KeyError, match="experts.1.w2.scale_weight"):
        C.load_moe_layers(bad, prefix=PRE)
    bad = dict(sd)
    bad[layer + ".experts.1.w2.weight"] = bad[layer + ".experts.1.w2.weight"][:, :-8].contiguous()
    with pytest.raises(ValueError, match="experts.1.w2.weight"):
        C.load_moe_layers(bad, prefix=PRE)
    bad = dict(sd)
    bad[layer + ".experts.0.w1.weight"] = bad[layer + ".experts.0.w1.weight"].to(BF16)   # unquantised weight, fp8 marker
    with pytest.raises(TypeError, match="experts.0.w1.weight"):
        C.load_moe_layers(bad, prefix=PRE)


def test_save_then_load_round_trip(tmp_path):
    sd = model_state_dict("fp8", layers=("double_stream_blocks.0.block.ff_i",))
    sd[PRE + "scaled_fp8"] = C.scaled_fp8_marker(FP8)
    modules, info = C.load_moe_layers(sd, prefix=PRE)
    path = os.path.join(tmp_path, "again.safetensors")
    keys = C.save_moe_layers(modules, path, prefix=PRE, scaled_fp8=info["scaled_fp8"],
                             fp8_optimizations=info["fp8_optimizations"])
    assert PRE + "scaled_fp8" in keys
    again, info2 = C.load_moe_layers(path, prefix=PRE)
    assert info2["scaled_fp8"] == FP8 and info2["fp8_optimizations"] is True
    for layer in modules:
        a, b = modules[layer].state_dict(), again[layer].state_dict()
        assert sorted(a) == sorted(b)
        for k in a:
            va, vb = a[k], b[k]
            if va.dtype == FP8:
                va, vb = va.view(torch.uint8), vb.view(torch.uint8)
            assert torch.equal(va, vb), k
