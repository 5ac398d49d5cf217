"""Pins the restatement of the scaled-fp8 weight maintenance path: stochastic rounding to float8_e4m3fn
(/root/reference/comfy/float.py:14-67 behind /root/reference/comfy/ops.py:419-426)."""
import os
import subprocess

import pytest
import torch

from oracle import hidream_moe_oracle as O

FP8 = torch.float8_e4m3fn
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# known-answer vectors of Philox4x32-10 from the Random123 distribution (kat_vectors): counter, key -> output
PHILOX_KAT = [
    ([0, 0, 0, 0], [0, 0], [0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8]),
    ([0xffffffff] * 4, [0xffffffff] * 2, [0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd]),
    ([0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344], [0xa4093822, 0x299f31d0],
     [0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1]),
]


def test_philox_known_answers_checker_and_product_header(tmp_path):
    for ctr, key, want in PHILOX_KAT:
        assert O.philox4x32_10(ctr, key) == want
    # the header the kernels include, built for the host
    src = tmp_path / "kat.c"
    lines = []
    for ctr, key, _ in PHILOX_KAT:
        lines.append("{ uint32_t c[4] = {%s}, k[2] = {%s}, o[4]; hdmoe_philox4x32_10(c, k, o); "
                     'printf("%%08x %%08x %%08x %%08x\\n", o[0], o[1], o[2], o[3]); }'
                     % (", ".join("0x%xu" % v for v in ctr), ", ".join("0x%xu" % v for v in key)))
    src.write_text('#include <stdio.h>\n#include "philox.h"\nint main(void) {\n' + "\n".join(lines) + "\nreturn 0; }\n")
    exe = tmp_path / "kat"
    subprocess.check_call(["gcc", "-std=c11", "-I", os.path.join(ROOT, "comfyui_amd", "csrc"), str(src), "-o", str(exe)])
    got = [[int(w, 16) for w in l.split()] for l in subprocess.check_output([str(exe)], text=True).splitlines()]
    assert got == [want for _, _, want in PHILOX_KAT]


def all_finite_codes():
    codes = torch.arange(256, dtype=torch.uint8)
    vals = codes.view(FP8).float()
    keep = ~vals.isnan()
    return codes[keep], vals[keep]


def test_representable_values_are_fixed_points_for_every_seed():
    codes, vals = all_finite_codes()
    for seed in (0, 1, 12345, 2 ** 40 + 3):
        out = O.stochastic_round_e4m3fn(vals, None, seed)
        got = out.view(torch.uint8)
        # -0.0 is an exact zero: the reference multiplies by sign(0) = 0, which gives +0
        want = torch.where(vals == 0, torch.zeros_like(codes), codes)
        assert torch.equal(got, want)


def neighbours(h):
    """Lower and upper e4m3fn neighbours (by magnitude) of float16-valued magnitudes h < 448, in float64."""
    _, vals = all_finite_codes()
    grid = torch.unique(vals[vals >= 0]).double()
    idx = torch.searchsorted(grid, h.double(), right=True) - 1
    lo = grid[idx]
    hi = grid[torch.clamp(idx + 1, max=grid.numel() - 1)]
    return lo, hi


def test_lands_on_a_neighbour_with_probability_equal_to_the_position():
    g = torch.Generator().manual_seed(0)
    # magnitudes over all binades incl. subnormal ones, both signs
    mags = torch.exp2(torch.rand(64, generator=g) * 17 - 10.5)      # 2^-10.5 .. 2^6.5
    x = (mags * torch.where(torch.rand(64, generator=g) < 0.5, -1.0, 1.0)).float()
    reps = 4096
    xs = x.repeat_interleave(reps)                                   # different element index -> different draw
    out = O.stochastic_round_e4m3fn(xs, None, seed=99).float().view(64, reps)
    h = x.half().float()
    lo, hi = neighbours(h.abs())
    sign = torch.sign(h).double().unsqueeze(1)
    o = out.double() * sign                                          # magnitudes
    assert bool(((o == lo.unsqueeze(1)) | (o == hi.unsqueeze(1))).all())
    p_want = torch.where(hi > lo, (h.abs().double() - lo) / (hi - lo), torch.zeros_like(lo))
    p_got = (o == hi.unsqueeze(1)).double().mean(dim=1)
    p_got = torch.where(hi > lo, p_got, torch.zeros_like(p_got))
    sigma = torch.sqrt(p_want * (1 - p_want) / reps) + 1e-3
    assert bool(((p_got - p_want).abs() < 5 * sigma).all()), (p_got - p_want).abs().max()
    # a plausible mistake (e.g. rounding to nearest, or a position measured in the wrong binade) fails this
    nearest = (p_want > 0.5).double()
    assert ((nearest - p_want).abs() > 5 * sigma).float().mean() > 0.8


def test_saturation_zero_and_sign_rules():
    x = torch.tensor([448.0, 449.0, 464.0, 480.0, 1e4, 7e4, float("inf"), -500.0, -float("inf")])
    out = O.stochastic_round_e4m3fn(x, None, 5).float()
    assert out.tolist() == [448.0] * 7 + [-448.0] * 2
    z = O.stochastic_round_e4m3fn(torch.tensor([0.0, -0.0]), None, 5).view(torch.uint8)
    assert z.tolist() == [0, 0]
    # a tiny negative value that rounds down to zero keeps its sign (sign * 0 in the reference's arithmetic)
    tiny = torch.full((64,), -1e-6)
    codes = O.stochastic_round_e4m3fn(tiny, None, 1).view(torch.uint8)
    assert set(codes.tolist()) <= {0x80, 0x81} and 0x80 in codes.tolist()
    assert bool(O.stochastic_round_e4m3fn(torch.tensor([float("nan")]), None, 0).float().isnan().all())
    # values between 416 and 448 go to one of the two, values in [448, 480) always to 448 (480 is not a value)
    hi = O.stochastic_round_e4m3fn(torch.full((256,), 440.0), None, 3).float()
    assert set(hi.tolist()) == {416.0, 448.0}


def test_value_is_rounded_to_float16_first():
    # 1 + 2^-12 is not a float16 value: it becomes exactly 1.0 and never rounds up; 1 + 2^-10 is one and does, rarely
    x = torch.full((1 << 16,), 1.0 + 2.0 ** -12)
    assert bool((O.stochastic_round_e4m3fn(x, None, 2).float() == 1.0).all())
    y = torch.full((1 << 16,), 1.0 + 2.0 ** -10)
    up = (O.stochastic_round_e4m3fn(y, None, 2).float() == 1.125).float().mean().item()
    assert 0.004 < up < 0.012                                         # position 2^-10 / 2^-3 = 1/128


def test_division_by_scale_and_bf16_source():
    g = torch.Generator().manual_seed(3)
    w = torch.randn(4096, generator=g)
    s = torch.tensor(0.25)
    assert torch.equal(O.stochastic_round_e4m3fn(w, s, 8).view(torch.uint8),
                       O.stochastic_round_e4m3fn(w * 4, None, 8).view(torch.uint8))
    # bf16 weights: the scale and the quotient are bf16 tensors in the reference's division
    s3 = torch.tensor(0.3)
    wb = w.to(torch.bfloat16)
    want_in = (wb / s3.to(torch.bfloat16)).float()
    assert torch.equal(O.stochastic_round_e4m3fn(wb, s3, 8).view(torch.uint8),
                       O.stochastic_round_e4m3fn(want_in, None, 8).view(torch.uint8))


def test_same_seed_same_bytes_other_seed_other_bytes():
    g = torch.Generator().manual_seed(4)
    w = torch.randn(10000, generator=g)
    a = O.stochastic_round_e4m3fn(w, None, 7).view(torch.uint8)
    assert torch.equal(a, O.stochastic_round_e4m3fn(w, None, 7).view(torch.uint8))
    assert not torch.equal(a, O.stochastic_round_e4m3fn(w, None, 8).view(torch.uint8))
    # element i depends on (value, seed, i) only: a prefix of the tensor gives a prefix of the result
    assert torch.equal(a[:1001], O.stochastic_round_e4m3fn(w[:1001], None, 7).view(torch.uint8))
