"""comfyui_amd.float_round.stochastic_rounding on host tensors against known answers recorded from the reference's
comfy/float.py:14-67 (tests/golden/make_float_round_golden.py, run once where the reference is present): the output
BYTES must be identical, i.e. the same float16 arithmetic and the same consumption order of the torch generator,
including across the slices of a tensor with more than 4096 * 4096 elements."""
import hashlib
import json
import os

import pytest
import torch
from safetensors.torch import load_file

from comfyui_amd import float_round

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DTYPES = {"e4m3fn": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2}


def test_small_cases_are_byte_identical():
    data = load_file(os.path.join(GOLDEN, "float_round.safetensors"))
    names = sorted(k[:-3] for k in data if k.endswith(".in"))
    assert len(names) == 5
    checked = 0
    for name in names:
        value = data[name + ".in"]
        for tag, dtype in DTYPES.items():
            for seed in (0, 1, 12345):
                want = data[f"{name}.{tag}.seed{seed}"]
                before = value.clone()
                got = float_round.stochastic_rounding(value, dtype, seed=seed)
                assert got.dtype == dtype and got.shape == value.shape
                assert torch.equal(value, before), "the input must not be modified"
                assert torch.equal(got.view(torch.uint8), want), (name, tag, seed)
                checked += 1
    assert checked == 30
    # different seeds give different bytes (the vectors are not degenerate), same seed the same bytes
    a = data["weights_f32.e4m3fn.seed0"]
    assert not torch.equal(a, data["weights_f32.e4m3fn.seed1"])


@pytest.mark.parametrize("tag", ["e4m3fn", "e5m2"])
def test_tensor_larger_than_one_slice(tag):
    big = json.load(open(os.path.join(GOLDEN, "float_round_big.json")))
    shape = tuple(big["shape"])
    assert shape[0] * shape[1] > 4096 * 4096
    g = torch.Generator().manual_seed(big["input_seed"])
    value = torch.randn(shape, generator=g) * 30
    case = big["cases"][tag]
    got = float_round.stochastic_rounding(value, DTYPES[tag], seed=case["seed"]).view(torch.uint8).reshape(-1)
    b = got.numpy().tobytes()
    assert list(b[:64]) == case["first64"]
    assert list(b[-64:]) == case["last64"], "the second slice continues the same generator stream"
    assert hashlib.sha256(b).hexdigest() == case["sha256"]
