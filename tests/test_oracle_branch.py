"""Pins the restatement of a block's feed-forward branch around the layer
(/root/reference/comfy/ldm/hidream/model.py:429-433, 515-523): LayerNorm + adaLN modulation in
front, gated residual behind."""
import pytest
import torch
import torch.nn.functional as F

from oracle import hidream_moe_oracle as O

BF16 = torch.bfloat16


def bf16_steps(a, b):
    """Distance in representable bf16 values between two bf16 tensors (monotone integer key)."""
    def key(t):
        i = t.view(torch.int16).to(torch.int32)
        return torch.where(i < 0, -(i & 0x7FFF), i)
    return (key(a) - key(b)).abs()


def make(B, S, D, seed, mean=0.0, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    x = (torch.randn((B, S, D), generator=g) * spread + mean).to(BF16)
    shift = (torch.randn((B, 1, D), generator=g) * 0.3).to(BF16)
    scale = (torch.randn((B, 1, D), generator=g) * 0.3).to(BF16)
    gate = (torch.randn((B, 1, D), generator=g) * 0.5).to(BF16)
    return x, shift, scale, gate


@pytest.mark.parametrize("B,S,D", [(1, 5, 8), (2, 33, 512), (3, 17, 2560), (1, 7, 520), (4, 1, 1024)])
def test_ln_modulate_fixed_order_agrees_with_torch_to_one_bf16_step(B, S, D):
    x, shift, scale, _ = make(B, S, D, seed=B * 1000 + D, mean=0.25, spread=1.5)
    want = O.ln_modulate_torch(x, shift, scale)
    got = O.ln_modulate_c(x.reshape(-1, D), shift.reshape(B, D), scale.reshape(B, D), S).view(B, S, D)
    # The statistics are fp32 sums in two different orders: the normalised value can land on the other side of a
    # rounding boundary for a few elements (one step, 2^-7 relative at most); the product then moves by that much
    # plus its own rounding step, the sum by one more step of its own. Everything else must be identical.
    n_want = F.layer_norm(x, (D,), None, None, 1e-6)
    assert n_want.dtype == BF16
    steps = bf16_steps(got, want)
    exact = (steps == 0).float().mean().item()
    assert exact > 0.98, exact
    err = (got.float() - want.float()).abs()
    bound = torch.maximum((n_want.float() * (1 + scale).float()).abs(), want.float().abs()) * (3 * 2.0 ** -7)
    assert bool((err <= bound + 1e-30).all())


def test_ln_modulate_closed_forms():
    # (a) a row of two alternating values +-a has mean 0 and variance a^2: normalised values are +-1 (eps-corrected)
    D = 512
    a = 3.0
    x = torch.tensor([a, -a] * (D // 2)).to(BF16).view(1, D)
    zero = torch.zeros((1, D), dtype=BF16)
    out = O.ln_modulate_c(x, zero, zero, 1, eps=0.0)
    assert torch.equal(out, torch.tensor([1.0, -1.0] * (D // 2)).to(BF16).view(1, D))
    # (b) with n = +-1 exactly: out = +-(1 + scale) + shift, rounded as bf16 ops
    g = torch.Generator().manual_seed(5)
    scale = torch.randn((1, D), generator=g).to(BF16)
    shift = torch.randn((1, D), generator=g).to(BF16)
    want = (out * (1 + scale)) + shift
    got = O.ln_modulate_c(x, shift, scale, 1, eps=0.0)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # (c) a constant row: variance 0, everything rests on eps; n = 0 so out = shift
    x = torch.full((1, D), 2.5).to(BF16)
    got = O.ln_modulate_c(x, shift, scale, 1, eps=1e-6)
    assert torch.equal(got.view(torch.int16), (torch.zeros_like(shift) * (1 + scale) + shift).view(torch.int16))
    # (d) shift invariance: adding a constant (exactly representable) to the row leaves n unchanged
    base = torch.tensor([1.0, -1.0, 2.0, -2.0] * (D // 4)).to(BF16).view(1, D)
    o1 = O.ln_modulate_c(base, zero, zero, 1)
    o2 = O.ln_modulate_c(base + 4.0, zero, zero, 1)
    assert torch.equal(o1, o2)
    # (e) batch rows: token t takes modulation row t // tokens_per_batch
    xs = torch.randn((6, D), generator=g).to(BF16)
    sc2 = torch.randn((2, D), generator=g).to(BF16)
    sh2 = torch.randn((2, D), generator=g).to(BF16)
    whole = O.ln_modulate_c(xs, sh2, sc2, 3)
    for b in range(2):
        part = O.ln_modulate_c(xs[3 * b:3 * b + 3], sh2[b:b + 1], sc2[b:b + 1], 3)
        assert torch.equal(whole[3 * b:3 * b + 3], part)


def test_ln_modulate_uses_biased_variance_and_eps_inside_the_root():
    # brute force in float64 for one short row; a plausible mistake (n-1 divisor, eps outside the root) moves the
    # result by several bf16 steps, the restatement stays within one
    g = torch.Generator().manual_seed(9)
    D = 8
    zero = torch.zeros((1, D), dtype=BF16)

    def f64(x, eps, divisor, eps_inside=True):
        xd = x.double()
        mean = xd.mean()
        var = ((xd - mean) ** 2).sum() / divisor
        den = torch.sqrt(var + eps) if eps_inside else torch.sqrt(var) + eps
        return ((xd - mean) / den).to(BF16)

    x = torch.randn((1, D), generator=g).to(BF16)
    got = O.ln_modulate_c(x, zero, zero, 1, eps=0.0)
    assert bool((bf16_steps(got, f64(x, 0.0, D)) <= 1).all())
    assert int((bf16_steps(got, f64(x, 0.0, D - 1)) > 4).sum()) >= D - 1          # sqrt(8/7): 6.9 % off

    x = (torch.randn((1, D), generator=g) * 0.01).to(BF16)                         # variance 1e-4, eps 1e-3
    got = O.ln_modulate_c(x, zero, zero, 1, eps=1e-3)
    assert bool((bf16_steps(got, f64(x, 1e-3, D)) <= 1).all())
    assert int((bf16_steps(got, f64(x, 1e-3, D, eps_inside=False)) > 4).sum()) >= D - 1


def test_gated_residual_matches_torch_bf16_expression_bit_for_bit():
    B, S, D = 3, 29, 640
    x, _, _, gate = make(B, S, D, seed=3)
    g = torch.Generator().manual_seed(4)
    y = torch.randn((B, S, D), generator=g).to(BF16)
    want = O.gated_residual_torch(y, gate, x)                      # model.py:432-433 at bf16
    got = O.gated_residual_c(y.reshape(-1, D), gate.reshape(B, D), x.reshape(-1, D), S).view(B, S, D)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_ff_branch_reduces_to_the_layer_and_to_identity():
    from comfyui_amd import synth
    master, _ = synth.make_weights(seed=21, dim=256, hidden_arg=256, num_experts=2)
    params = O.oracle_params(synth.to_state_dict(master, "bf16"), 2)
    B, S, D = 2, 24, 256
    x, shift, scale, gate = make(B, S, D, seed=8)
    out, n = O.ff_branch(x, shift, scale, gate, params, "plain")
    # gate = 0: the branch is the identity on x
    out0, _ = O.ff_branch(x, shift, scale, torch.zeros_like(gate), params, "plain")
    assert torch.equal(out0, x)
    # the branch is the layer applied to the normalised tokens, gated, plus x
    y = O.moe_forward(n, params, "plain")
    assert torch.equal(out, gate * y + x)
    # fixed-order statistics change the normalised tokens by at most one step on few elements
    _, n2 = O.ff_branch(x, shift, scale, gate, params, "plain", fixed_order_norm=True)
    assert (bf16_steps(n, n2) == 0).float().mean().item() > 0.98
