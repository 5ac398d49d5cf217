"""Seeded sweep over layer shapes the fixed cases do not name: width, expert count (2..16), hidden widths, ragged
token counts around the tile heights, batch split, both weight types, per-Linear scale_input values. Every case:
routing bit-exact against the fixed-order oracle, output against the oracle's bf16-dataflow restatement of
MOEFeedForwardSwiGLU.forward (/root/reference/comfy/ldm/hidream/model.py:307-325) at half the stated tolerance."""
import random

import pytest
import torch

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16
TOL = {"fp8": 3e-2, "bf16": 1e-2}


def _cases(seed, n):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        dim = rng.choice([256, 512, 768, 1024])
        T = rng.choice([1, 2, 7, 63, 64, 65, 255, 256, 257, 300, 511, 700, 1023, 1025, 1500, 2049])
        out.append(dict(dim=dim, E=rng.choice([2, 3, 4, 4, 4, 5, 8, 16]),
                        hidden_arg=rng.choice([dim, 2 * dim, 4 * dim, 6 * dim]), T=T,
                        batch=rng.choice([1, 1, 2]) if T % 2 == 0 else 1, weights=rng.choice(["fp8", "fp8", "bf16"]),
                        seed=rng.randrange(10000), scales=rng.random() < 0.5, pick=rng.randrange(1 << 30)))
    return out


@pytest.mark.parametrize("case", _cases(20240607, 40), ids=lambda c: f"d{c['dim']}-E{c['E']}-h{c['hidden_arg']}-T{c['T']}-{c['weights']}")
def test_random_layer(dev, case):
    from comfyui_amd import functional as HF
    dim, E, weights = case["dim"], case["E"], case["weights"]
    master, g = synth.make_weights(case["seed"], dim=dim, hidden_arg=case["hidden_arg"], num_experts=E)
    sd = synth.to_state_dict(master, weights)
    if weights == "fp8" and case["scales"]:
        rng = random.Random(case["pick"])
        for k in list(sd):
            if k.endswith("w1.scale_input"):
                v = torch.tensor(rng.choice([0.5, 1.0, 0.37, 2.0]), dtype=torch.float32)
                sd[k] = v
                sd[k.replace("w1.", "w3.")] = v.clone()
            elif k.endswith("w2.scale_input"):
                sd[k] = torch.tensor(rng.choice([0.5, 1.0, 0.81]), dtype=torch.float32)
    x = synth.make_input(g, case["T"], dim=dim, batch=case["batch"])
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=dim, hidden_arg=case["hidden_arg"],
                           num_experts=E)
    xd = x.to(dev)
    y = m(xd)
    idx, w = HF.gate_top2(xd.reshape(-1, dim), m.gate.weight.to(BF16))
    torch.cuda.synchronize()
    y, idx, w = y.cpu(), idx.cpu(), w.cpu()
    x2 = x.reshape(-1, dim)
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x2, sd["gate.weight"])
    assert torch.equal(idx, idx_ref) and torch.equal(w.view(torch.int16), w_ref.view(torch.int16))
    ref = O.moe_forward(x2.unsqueeze(0), O.oracle_params(sd, E), "fp8mm" if weights == "fp8" else "plain",
                        gate_result=(idx, w))
    met = O.error_metrics(y.reshape(1, -1, dim), ref)
    assert y.shape == x.shape and not bool(y.float().isnan().any())
    assert met["rel_rms"] <= TOL[weights] / 2 and met["max_over_max"] <= TOL[weights], met
