"""Writes tests/golden/float_round.safetensors (+ float_round_big.json): known answers of the reference's
stochastic rounding to fp8 for host tensors.

Run in the build container only (the reference is not present anywhere else):
    python tests/golden/make_float_round_golden.py

It loads /root/reference/comfy/float.py by file path (that file imports nothing but torch) and records
stochastic_rounding(value, dtype, seed) for CPU tensors:
  * small cases, stored whole (inputs and output bytes): every binade of both fp8 formats, subnormals, zeros of both
    signs, values beyond the largest finite fp8 number, float32 / bfloat16 / float16 sources, several seeds,
    1-D and 2-D shapes;
  * one large case per format whose element count exceeds 4096 * 4096, so that the reference's slice loop
    (float.py:58-65) runs twice and the generator is consumed across slices. Its input is regenerated from a seed by
    the test; the fixture holds the SHA-256 of the output bytes and the first and last 64 of them.
tests/test_float_round_golden.py compares comfyui_amd.float_round.stochastic_rounding with these byte for byte.
"""
import hashlib
import importlib.util
import json
import os

import torch
from safetensors.torch import save_file

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE = "/root/reference/comfy/float.py"
BIG_SHAPE = (5000, 4096)      # 20.48 M elements: two slices (4096 rows, then 904)
BIG_SEED_INPUT = 1234


def small_inputs():
    g = torch.Generator().manual_seed(7)
    cases = {}
    # all binades of e5m2 (2^-16 .. 2^15) and beyond, both signs, random mantissas
    exps = torch.arange(-20, 18, dtype=torch.float32)
    mant = 1.0 + torch.rand((exps.numel(), 24), generator=g)
    sign = torch.where(torch.rand(mant.shape, generator=g) < 0.5, -1.0, 1.0)
    spread = (sign * mant * torch.exp2(exps)[:, None]).reshape(-1)
    special = torch.tensor([0.0, -0.0, 448.0, -448.0, 449.0, 464.0, 480.0, 500.0, -1000.0, 57344.0, 60000.0, 65504.0,
                            2.0 ** -9, 2.0 ** -10, 2.0 ** -7, 2.0 ** -6, 1.0, -1.0, 0.0625, 1.5, 3.0e-5, 1.0e-8])
    cases["spread_f32"] = torch.cat([spread, special])
    cases["weights_f32"] = torch.randn((96, 80), generator=g) * 0.02 / 0.00021     # a weight matrix over its scale
    cases["weights_bf16"] = (torch.randn((64, 48), generator=g) * 3.0).to(torch.bfloat16)
    cases["weights_f16"] = (torch.randn((33, 17), generator=g) * 40.0).to(torch.float16)
    cases["one_row"] = torch.randn((1, 257), generator=g) * 100.0
    return cases


def main():
    spec = importlib.util.spec_from_file_location("reference_float", REFERENCE)
    ref = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(ref)
    out = {}
    for name, value in small_inputs().items():
        out[f"{name}.in"] = value.contiguous()
        for dtype, tag in ((torch.float8_e4m3fn, "e4m3fn"), (torch.float8_e5m2, "e5m2")):
            for seed in (0, 1, 12345):
                r = ref.stochastic_rounding(value.clone(), dtype, seed=seed)
                out[f"{name}.{tag}.seed{seed}"] = r.view(torch.uint8).contiguous()
    save_file(out, os.path.join(HERE, "float_round.safetensors"))
    big = {"shape": list(BIG_SHAPE), "input_seed": BIG_SEED_INPUT, "input": "torch.randn(shape, generator=Generator().manual_seed(input_seed)) * 30", "cases": {}}
    g = torch.Generator().manual_seed(BIG_SEED_INPUT)
    value = torch.randn(BIG_SHAPE, generator=g) * 30
    for dtype, tag in ((torch.float8_e4m3fn, "e4m3fn"), (torch.float8_e5m2, "e5m2")):
        r = ref.stochastic_rounding(value, dtype, seed=3).view(torch.uint8).reshape(-1)
        b = r.numpy().tobytes()
        big["cases"][tag] = {"seed": 3, "sha256": hashlib.sha256(b).hexdigest(), "first64": list(b[:64]), "last64": list(b[-64:])}
    with open(os.path.join(HERE, "float_round_big.json"), "w") as f:
        json.dump(big, f, indent=1)
    print("wrote", len(out), "tensors and the large-case digests")


if __name__ == "__main__":
    main()
