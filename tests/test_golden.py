"""The committed fixture tests/golden/moe_small.safetensors (written by tests/golden/make_golden.py from the CPU
oracle) against the oracle (CPU) and against the HIP path (GPU)."""
import os

import pytest
import torch
from safetensors.torch import load_file

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "moe_small.safetensors")
DIM, HIDDEN_ARG, E = 256, 384, 2
FP8 = torch.float8_e4m3fn


def load(weights):
    t = load_file(PATH)
    pre = weights + "."
    d = {k[len(pre):]: v for k, v in t.items() if k.startswith(pre)}
    sd = {}
    for k, v in d.items():
        if k.startswith("sd."):
            sd[k[3:]] = v.view(FP8) if v.dtype == torch.uint8 else v
    return d, sd


@pytest.mark.parametrize("weights", ["fp8", "bf16"])
def test_oracle_reproduces_fixture(weights):
    d, sd = load(weights)
    x2 = d["x"].reshape(-1, DIM)
    idx, w, logits, scores = O.gate_fixed_order(x2, sd["gate.weight"])
    assert torch.equal(idx, d["topk_idx"]) and torch.equal(w.view(torch.int16), d["topk_weight"].view(torch.int16))
    ties = d["scores"][::6]
    assert bool((ties[:, 0] == ties[:, 1]).all()) and d["topk_idx"][::6].tolist() == [[0, 1]] * 8
    counts, offsets, perm, inv = O.dispatch(idx, E)
    assert torch.equal(perm, d["perm"]) and torch.equal(offsets, d["offsets"])
    y = O.moe_forward(d["x"], O.oracle_params(sd, E), "fp8mm" if weights == "fp8" else "plain", gate_result=(idx, w))
    assert O.error_metrics(y, d["y"])["rel_rms"] < 1e-3      # torch's CPU matmul blocking may differ between hosts


@pytest.mark.gpu
@pytest.mark.parametrize("weights", ["fp8", "bf16"])
def test_hip_path_against_fixture(dev, weights):
    from comfyui_amd import functional as HF
    d, sd = load(weights)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=DIM, hidden_arg=HIDDEN_ARG,
                           num_experts=E)
    x = d["x"].to(dev)
    y = m(x).cpu()
    idx, w = HF.gate_top2(x.reshape(-1, DIM), m.gate.weight)
    assert torch.equal(idx.cpu(), d["topk_idx"])
    assert torch.equal(w.cpu().view(torch.int16), d["topk_weight"].view(torch.int16))
    counts, offsets, perm, inv = HF.dispatch(idx, E)
    assert torch.equal(perm.cpu(), d["perm"]) and torch.equal(inv.cpu(), d["inv_perm"])
    assert torch.equal(counts.cpu(), d["counts"]) and torch.equal(offsets.cpu(), d["offsets"])
    met = O.error_metrics(y, d["y"])
    print(weights, met)
    assert met["rel_rms"] <= (1e-2 if weights == "fp8" else 4e-3) and met["max_over_max"] <= 3e-2
