"""Pins the restatement of the Hunyuan3D-2.1 MoEBlock
(/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:8-188, inference branch)."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import hidream_moe_oracle as O
from tests.test_oracle_branch import bf16_steps

BF16 = torch.bfloat16


def make_block(dim, inner, E, seed, dtype=BF16, bias_scale=0.5):
    g = torch.Generator().manual_seed(seed)
    sd = {}

    def ff(prefix):
        sd[prefix + "net.0.proj.weight"] = (torch.randn((inner, dim), generator=g) / math.sqrt(dim)).to(dtype)
        sd[prefix + "net.0.proj.bias"] = (torch.randn((inner,), generator=g) * bias_scale).to(dtype)
        sd[prefix + "net.2.weight"] = (torch.randn((dim, inner), generator=g) / math.sqrt(inner)).to(dtype)
        sd[prefix + "net.2.bias"] = (torch.randn((dim,), generator=g) * bias_scale).to(dtype)

    for e in range(E):
        ff(f"experts.{e}.")
    ff("shared_experts.")
    sd["gate.weight"] = (torch.randn((E, dim), generator=g) / math.sqrt(dim)).to(dtype)
    return sd, g


def test_linear_bias_single_rounding_agrees_with_torch_bf16_linear():
    g = torch.Generator().manual_seed(0)
    x = torch.randn((64, 256), generator=g).to(BF16)
    w = (torch.randn((128, 256), generator=g) / 16).to(BF16)
    b = torch.randn((128,), generator=g).to(BF16)
    got = O.linear_bias(x, w, b)
    want = F.linear(x, w, b)
    steps = bf16_steps(got, want)
    assert int(steps.max()) <= 1 and (steps == 0).float().mean().item() > 0.99
    # closed form in float64: one rounding of the exact sum
    exact = (x.double() @ w.double().t() + b.double())
    assert int(bf16_steps(got, exact.to(BF16)).max()) <= 1
    assert torch.equal(O.linear_bias(x, w, None), (x.float() @ w.float().t()).to(BF16))
    # a dropped or doubled bias is far outside one step
    assert int(bf16_steps(O.linear_bias(x, w, None), want).max()) > 8


def test_gelu_is_the_erf_form_rounded_once():
    x = torch.linspace(-6, 6, 4001).to(BF16)
    want = (0.5 * x.double() * (1 + torch.erf(x.double() / math.sqrt(2)))).to(BF16)
    got = F.gelu(x)
    # torch evaluates 1 + erf(.) in fp32, which cancels to 0 below x = -5.5 where the true value is ~1e-8
    core = x.float().abs() <= 4
    assert int(bf16_steps(got[core], want[core]).max()) <= 1
    assert float((got.float() - want.float()).abs().max()) < 1e-6 + 2.0 ** -8 * 6
    tanh_form = F.gelu(x, approximate="tanh")
    assert int(bf16_steps(tanh_form[core], want[core]).max()) > 1   # the other GELU is distinguishable at bf16


def test_feed_forward_closed_forms():
    dim, inner = 64, 256
    sd, g = make_block(dim, inner, 1, seed=2)
    ff = O.hunyuan_params(sd, 1)["shared"]
    x = torch.randn((8, dim), generator=g).to(BF16)
    # zero input: out = W_out gelu(b_in) + b_out
    zero = torch.zeros((1, dim), dtype=BF16)
    want = O.linear_bias(F.gelu(ff[1].unsqueeze(0)), ff[2], ff[3])
    assert torch.equal(O.gelu_feed_forward(zero, ff), want)
    # against float64 end to end within bf16 accuracy of a 256-term sum
    w_in, b_in, w_out, b_out = (t.double() for t in ff)
    h = F.linear(x.double(), w_in, b_in)
    ref = F.linear(0.5 * h * (1 + torch.erf(h / math.sqrt(2))), w_out, b_out)
    got = O.gelu_feed_forward(x, ff).double()
    assert ((got - ref).norm() / ref.norm()).item() < 1e-2


@pytest.mark.parametrize("E", [6, 8])
def test_block_equals_dense_brute_force_and_handles_empty_experts(E):
    dim, inner, T = 64, 256, 96
    sd, g = make_block(dim, inner, E, seed=E)
    params = O.hunyuan_params(sd, E)
    x = torch.randn((2, T // 2, dim), generator=g).to(BF16)
    idx, w, _, _ = O.gate_torch(x.reshape(-1, dim), params["gate"])
    y = O.hunyuan_moe_block(x, params)
    # the index_add_ accumulation in expert order rounds like the two-term slot sum (addition commutes)
    assert torch.equal(y, O.hunyuan_moe_block_dense(x, params, idx, w))
    # routing that never uses some experts
    idx2 = torch.stack([torch.zeros(T, dtype=torch.long), torch.full((T,), E - 1, dtype=torch.long)], dim=1)
    y2 = O.hunyuan_moe_block(x, params, gate_result=(idx2, w))
    assert torch.equal(y2, O.hunyuan_moe_block_dense(x, params, idx2, w))
    # all experts identical: (w0 + w1 as separate roundings) * FF(x) + shared
    same = dict(params, experts=[params["experts"][0]] * E)
    ffx = O.gelu_feed_forward(x.reshape(-1, dim), params["experts"][0])
    want = ((ffx * w[:, 0:1]) + (ffx * w[:, 1:2])).view(x.shape) + O.gelu_feed_forward(x, params["shared"])
    assert torch.equal(O.hunyuan_moe_block(x, same, gate_result=(idx, w)), want)


def test_gate_for_six_experts_matches_fixed_order_restatement():
    dim, E, T = 512, 6, 300
    sd, g = make_block(dim, 256, E, seed=9)
    x = torch.randn((T, dim), generator=g).to(BF16)
    idx_t, w_t, _, _ = O.gate_torch(x, sd["gate.weight"])
    idx_c, w_c, _, _ = O.gate_fixed_order(x, sd["gate.weight"])
    agree = (idx_t == idx_c).all(dim=1).float().mean().item()
    assert agree > 0.99                                           # summation-order flips only
