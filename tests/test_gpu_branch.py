"""GPU parity of a block's feed-forward branch around the layer
(/root/reference/comfy/ldm/hidream/model.py:429-433, 515-523): LayerNorm + adaLN modulation kernel, the
gated-residual combine, and the one-enqueue branch (MOEFeedForwardSwiGLU.forward_branch)."""
import pytest
import torch

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O
from tests.helpers import oracle_params, small_layer
from tests.test_gpu_layer import TOL, TOL_RMS_SAME_DATAFLOW
from tests.test_oracle_branch import bf16_steps, make

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def bits(t):
    return t.view(torch.int16)


@pytest.mark.parametrize("B,S,D", [(1, 1, 2560), (2, 257, 2560), (3, 100, 512), (1, 77, 520), (2, 1, 8), (1, 3000, 2560)])
def test_ln_modulate_bit_exact(dev, B, S, D):
    from comfyui_amd import functional as HF
    x, shift, scale, _ = make(B, S, D, seed=B + S + D, mean=0.5, spread=2.0)
    want = O.ln_modulate_c(x.reshape(-1, D), shift.reshape(B, D), scale.reshape(B, D), S)
    got = HF.ln_modulate(x.reshape(-1, D).to(dev), scale.to(dev), shift.to(dev), S).cpu()
    assert torch.equal(bits(got), bits(want))


def test_ln_modulate_rejects_bad_shapes(dev):
    from comfyui_amd import functional as HF
    x, shift, scale, _ = make(2, 10, 512, seed=1)
    with pytest.raises(ValueError):
        HF.ln_modulate(x.reshape(-1, 512).to(dev), scale.to(dev), shift.to(dev), 7)
    with pytest.raises(RuntimeError):
        HF.ln_modulate(x.reshape(-1, 512), scale, shift, 10)          # CPU tensors: no CPU path


@pytest.mark.parametrize("T,D,B,with_shared", [(96, 640, 3, True), (1, 256, 1, True), (1000, 2560, 2, True),
                                               (130, 512, 5, False)])
def test_combine_gated_residual_bit_exact(dev, T, D, B, with_shared):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(T + D)
    S = T // B
    T = S * B
    y = torch.randn((2 * T, D), generator=g).to(BF16)
    w = torch.rand((T, 2), generator=g).to(BF16)
    sh = torch.randn((T, D), generator=g).to(BF16) if with_shared else None
    gate = (torch.randn((B, D), generator=g) * 0.5).to(BF16)
    res = torch.randn((T, D), generator=g).to(BF16)
    inv = torch.randperm(2 * T, generator=g).to(torch.int32)
    want = O.gated_residual_c(O.combine_c(y, inv, w, sh), gate, res, S)
    got = HF.combine_gated_residual(y.to(dev), inv.to(dev), w.to(dev), None if sh is None else sh.to(dev),
                                    gate.to(dev), res.to(dev), S).cpu()
    assert torch.equal(bits(got), bits(want))
    # and the torch expression the reference evaluates, at bf16
    ys = y[inv.long()].view(T, 2, D)
    ffn = (ys * w.unsqueeze(-1)).sum(dim=1)
    if sh is not None:
        ffn = ffn + sh
    want_torch = gate.view(B, 1, D) * ffn.view(B, S, D) + res.view(B, S, D)
    assert torch.equal(bits(got), bits(want_torch.reshape(T, D)))


@pytest.mark.parametrize("weights", ["fp8", "bf16"])
@pytest.mark.parametrize("dim,tokens,batch", [(256, 64, 1), (512, 700, 2), (1024, 513, 3)])
def test_branch_small_layers(dev, weights, dim, tokens, batch):
    from comfyui_amd import functional as HF
    S = tokens // batch
    sd, _ = small_layer(seed=dim + tokens, dim=dim, tokens=S * batch, weights=weights, batch=batch)
    x, shift, scale, gate = make(batch, S, dim, seed=tokens, mean=0.1, spread=1.3)
    # the synthetic layer's output is ~50x smaller than x: a large gate brings the feed-forward part up to the
    # size of the residual, so that the rounding of the sum does not hide it
    gate = (gate * 64).to(BF16)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=dim)
    out = m.forward_branch(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    assert out.shape == x.shape and out.dtype == BF16

    # the tokens the layer saw, and its routing on them: bit-exact against the fixed-order oracle
    n = O.ln_modulate_c(x.reshape(-1, dim), shift.reshape(batch, dim), scale.reshape(batch, dim), S)
    idx_ref, w_ref, _, _ = O.gate_fixed_order(n, sd["gate.weight"])
    idx, w = HF.gate_top2(n.to(dev), m.gate.weight.to(BF16))
    assert torch.equal(idx.cpu(), idx_ref) and torch.equal(bits(w.cpu()), bits(w_ref))

    params = oracle_params(sd, 4)
    mode = "fp8mm" if weights == "fp8" else "plain"
    ref, _ = O.ff_branch(x, shift, scale, gate, params, mode, gate_result=(idx_ref, w_ref), fixed_order_norm=True)
    # fp32 intermediates inside the layer and the residual, on the same bf16 normalised tokens. (With the LayerNorm
    # left unrounded as well, the reference's own bf16 dataflow is already 4e-2 away from the fp32 one on these
    # small layers: the fp8 quantisation of the layer input picks other codes. That is oracle against oracle.)
    ref32 = gate.float() * O.moe_forward(n.view(batch, S, dim).float(), params, mode,
                                         gate_result=(idx_ref, w_ref.float())) + x.float()
    # gate the whole branch and its feed-forward part (out - x) with the layer tests' tolerances
    delta, delta_ref, delta_ref32 = out.float() - x.float(), ref.float() - x.float(), ref32 - x.float()
    m_same = O.error_metrics(out, ref)
    m_delta = O.error_metrics(delta, delta_ref)
    m_delta32 = O.error_metrics(delta, delta_ref32)
    print(f"\n[{weights}] branch vs oracle {m_same}\n   ff part vs bf16 dataflow {m_delta}\n   ff part vs fp32 dataflow {m_delta32}")
    assert m_same["rel_rms"] <= TOL_RMS_SAME_DATAFLOW[weights]
    assert m_delta["rel_rms"] <= TOL[weights] and m_delta32["rel_rms"] <= TOL[weights]


@pytest.mark.parametrize("weights", ["fp8", "bf16"])
def test_branch_equals_its_three_stages(dev, weights):
    """One enqueue == ln_modulate -> layer -> torch's gate * y + x on the device, bit for bit; gate = 0 is the identity."""
    from comfyui_amd import functional as HF
    dim, B, S = 512, 2, 300
    sd, _ = small_layer(seed=5, dim=dim, tokens=B * S, weights=weights, batch=B)
    x, shift, scale, gate = (t.to(dev) for t in make(B, S, dim, seed=6))
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=dim)
    fused = m.forward_branch(x, shift, scale, gate)
    n = HF.ln_modulate(x.reshape(-1, dim), scale, shift, S).view(B, S, dim)
    staged = gate * m(n) + x
    assert torch.equal(bits(fused), bits(staged))
    assert torch.equal(m.forward_branch(x, shift, scale, torch.zeros_like(gate)), x)
    # composed path (mixed storage dtypes) gives the same branch
    m.experts[1].w2.hdmoe_fp8_matrix_mult = False
    composed = m.forward_branch(x, shift, scale, gate) if weights == "fp8" else None
    if composed is not None:
        d = O.error_metrics(composed.cpu(), fused.cpu())
        assert d["rel_rms"] < 1e-2, d


@pytest.mark.parametrize("B,S,E", [(3, 77, 4), (1, 1, 4), (2, 129, 2), (5, 13, 3)])
def test_branch_with_layernorm_inside_the_gate_kernel(dev, B, S, E):
    """At width 2560 with up to four fp8 experts the LayerNorm + modulation run inside the gate + cast kernel: the
    branch must still equal its three stages bit for bit (ragged token counts, several batch rows, 2..4 experts)."""
    from comfyui_amd import functional as HF
    dim, hidden_arg = 2560, 1024
    master, g = synth.make_weights(B * 100 + S, dim=dim, hidden_arg=hidden_arg, num_experts=E)
    sd = synth.to_state_dict(master, "fp8")
    for i, k in enumerate(sorted(k for k in sd if k.endswith("w1.scale_input"))):
        v = torch.tensor(0.5 + 0.25 * (i % 3), dtype=torch.float32)      # experts cast with different scales
        sd[k] = v
        sd[k.replace("w1.", "w3.")] = v.clone()
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev, dim=dim, hidden_arg=hidden_arg,
                           num_experts=E)
    x, shift, scale, gate = (t.to(dev) for t in make(B, S, dim, seed=S, mean=0.3, spread=1.7))
    fused = m.forward_branch(x, shift, scale, gate)
    n = HF.ln_modulate(x.reshape(-1, dim), scale, shift, S).view(B, S, dim)
    assert torch.equal(bits(fused), bits(gate * m(n) + x))


def test_branch_at_headline_size_properties(dev):
    """cfg3 shape (8192 tokens, fp8): gate = 0 is the identity, the fused branch equals its stages bit for bit,
    and the normalised tokens match torch's own layer_norm on the device to one bf16 step."""
    from comfyui_amd import functional as HF
    cfg = synth.make_config("cfg3")
    sd = synth.to_state_dict(cfg["master"], "fp8")
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, "fp8", dev)
    x = cfg["x"].to(dev)
    B, S, D = x.shape
    _, shift, scale, gate = (t.to(dev) for t in make(B, 1, D, seed=12))
    fused = m.forward_branch(x, shift, scale, gate)
    n = HF.ln_modulate(x.reshape(-1, D), scale, shift, S).view(B, S, D)
    assert torch.equal(bits(fused), bits(gate * m(n) + x))
    assert torch.equal(m.forward_branch(x, shift, scale, torch.zeros_like(gate)), x)
    ln = torch.nn.functional.layer_norm(x, (D,), None, None, 1e-6)
    n_torch = ln * (1 + scale) + shift
    steps = bf16_steps(n.cpu(), n_torch.cpu())
    assert (steps == 0).float().mean().item() > 0.98
    # statistics summed in another order can move the normalised value one step (2^-7 relative at most); the
    # product moves by that much plus its own rounding step, the sum by one more step of its own
    err = (n.float() - n_torch.float()).abs()
    bound = torch.maximum((ln.float() * (1 + scale).float()).abs(), n_torch.float().abs()) * (3 * 2.0 ** -7)
    assert bool((err <= bound + 1e-30).all())


@pytest.mark.parametrize("weights", ["fp8", "bf16"])
def test_dense_feed_forward_branch(dev, weights):
    """Text-stream branch: ln_modulate -> dense SwiGLU feed-forward -> gate and residual (model.py:518-523)."""
    from comfyui_amd import functional as HF
    dim, B, S = 512, 2, 130
    sd, _ = small_layer(seed=13, dim=dim, tokens=B * S, weights=weights, batch=B)
    x, shift, scale, gate = make(B, S, dim, seed=14)
    gate = (gate * 64).to(BF16)
    m = synth.build_module({k: v.to(dev) for k, v in sd.items()}, weights, dev, dim=dim)
    ff = m.shared_experts
    out = ff.forward_branch(x.to(dev), shift.to(dev), scale.to(dev), gate.to(dev)).cpu()
    # the gated residual kernel alone: bit-exact against the restatement and torch's bf16 expression
    g = torch.Generator().manual_seed(3)
    y = torch.randn((B * S, dim), generator=g).to(BF16)
    got = HF.gated_residual(y.to(dev), gate.to(dev), x.reshape(-1, dim).to(dev), S).cpu()
    assert torch.equal(bits(got), bits(O.gated_residual_c(y, gate.reshape(B, dim), x.reshape(-1, dim), S)))
    assert torch.equal(bits(got), bits((gate * y.view(B, S, dim) + x).reshape(-1, dim)))
    # the branch against the oracle's pieces
    params = oracle_params(sd, 4)
    mode = "fp8mm" if weights == "fp8" else "plain"
    n = O.ln_modulate_c(x.reshape(-1, dim), shift.reshape(B, dim), scale.reshape(B, dim), S).view(B, S, dim)
    ref = O.gated_residual_torch(O.ffn_swiglu(n, params["shared"], mode), gate, x)
    d_all = O.error_metrics(out, ref)
    d_ff = O.error_metrics(out.float() - x.float(), ref.float() - x.float())
    assert d_all["rel_rms"] <= TOL_RMS_SAME_DATAFLOW[weights] and d_ff["rel_rms"] <= TOL[weights], (d_all, d_ff)
    assert torch.equal(ff.forward_branch(x.to(dev), shift.to(dev), scale.to(dev), torch.zeros_like(gate).to(dev)).cpu(), x)
