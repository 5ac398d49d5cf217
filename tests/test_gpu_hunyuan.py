"""GPU parity of the Hunyuan3D-2.1 MoEBlock path (/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:8-188):
grouped Linear with bias and erf-GELU epilogue, the gate for 6 and 8 experts, and the whole block."""
import pytest
import torch

from oracle import hidream_moe_oracle as O
from tests.test_oracle_branch import bf16_steps
from tests.test_oracle_hunyuan import make_block

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def close_bf16(got, ref, frac_exact=0.97, rel=6e-3):
    """Same contraction in another summation order and erff of another library: nearly all elements identical,
    the rest within two steps of bf16 / a small fraction of the tensor's scale."""
    steps = bf16_steps(got, ref)
    err = (got.float() - ref.float()).abs()
    assert (steps == 0).float().mean().item() >= frac_exact, (steps == 0).float().mean().item()
    assert bool((err <= ref.float().abs() * 2.0 ** -6 + rel * ref.float().abs().mean()).all()), err.max()


@pytest.mark.parametrize("act", ["none", "gelu"])
@pytest.mark.parametrize("rows,K,N,bias", [(1, 256, 256, True), (300, 512, 768, True), (1025, 2048, 512, False)])
def test_single_linear_with_bias_and_gelu(dev, act, rows, K, N, bias):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(rows + K)
    x = torch.randn((rows, K), generator=g).to(BF16)
    w = (torch.randn((N, K), generator=g) / K ** 0.5).to(BF16)
    b = torch.randn((N,), generator=g).to(BF16) if bias else None
    ref = O.linear_bias(x, w, b)
    if act == "gelu":
        ref = torch.nn.functional.gelu(ref)
    xd = x.to(dev)
    _, got = HF.grouped_linear(xd[:0], None, [], a_static=xd, shared=(w.to(dev), None if b is None else b.to(dev)), act=act)
    close_bf16(got.cpu(), ref)


def test_grouped_linear_segments_with_empty_and_ragged_experts(dev):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(7)
    K, N, E = 256, 512, 6
    counts = [0, 37, 300, 0, 1, 257]
    rows = sum(counts)
    offsets = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
    a = torch.randn((rows, K), generator=g).to(BF16)
    ws = [((torch.randn((N, K), generator=g) / 16).to(BF16), torch.randn((N,), generator=g).to(BF16)) for _ in range(E)]
    xs = torch.randn((90, K), generator=g).to(BF16)
    wsh = ((torch.randn((N, K), generator=g) / 16).to(BF16), torch.randn((N,), generator=g).to(BF16))
    out, out_sh = HF.grouped_linear(a.to(dev), offsets.to(dev), [(w.to(dev), b.to(dev)) for w, b in ws],
                                    a_static=xs.to(dev), shared=(wsh[0].to(dev), wsh[1].to(dev)), act="gelu")
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            close_bf16(out[lo:hi].cpu(), torch.nn.functional.gelu(O.linear_bias(a[lo:hi], *ws[e])), frac_exact=0.95)
    close_bf16(out_sh.cpu(), torch.nn.functional.gelu(O.linear_bias(xs, *wsh)), frac_exact=0.95)


def test_bad_arguments(dev):
    from comfyui_amd import functional as HF
    x = torch.zeros((4, 256), dtype=BF16, device=dev)
    w = torch.zeros((256, 256), dtype=BF16, device=dev)
    with pytest.raises(KeyError):
        HF.grouped_linear(x[:0], None, [], a_static=x, shared=(w, None), act="relu")
    with pytest.raises(ValueError):
        HF.grouped_linear(x[:0], None, [], a_static=x, shared=(w[:, :128].contiguous(), None))
    with pytest.raises(Exception):
        HF.grouped_linear(x[:0], None, [], a_static=x, shared=(torch.zeros((200, 256), dtype=BF16, device=dev), None))


@pytest.mark.parametrize("E,dim,inner,tokens", [(8, 512, 2048, 700), (6, 256, 1024, 65), (8, 2048, 8192, 1500)])
def test_moe_block(dev, E, dim, inner, tokens):
    from comfyui_amd import functional as HF
    from comfyui_amd import hunyuan3d as H
    sd, g = make_block(dim, inner, E, seed=E + dim, bias_scale=0.2)
    x = torch.randn((1, tokens, dim), generator=g).to(BF16)
    m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, dtype=BF16, device=dev).eval()
    missing, unexpected = m.load_state_dict({k: v.to(dev) for k, v in sd.items()}, strict=True)
    y = m(x.to(dev)).cpu()
    assert y.shape == x.shape and y.dtype == BF16
    # routing: bit-exact against the fixed-order restatement, also through the module's gate
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    idx, w, aux = m.gate(x.to(dev))
    assert aux is None and idx.dtype == torch.int64
    assert torch.equal(idx.cpu(), idx_ref.long()) and torch.equal(w.cpu().view(torch.int16), w_ref.view(torch.int16))
    params = O.hunyuan_params(sd, E)
    ref = O.hunyuan_moe_block(x, params, gate_result=(idx_ref, w_ref))
    ref32 = O.hunyuan_moe_block(x.float(), {k: ([tuple(t.float() for t in ff) for ff in v] if k == "experts"
                                                  else (v.float() if k == "gate" else tuple(t.float() for t in v)))
                                             for k, v in params.items()}, gate_result=(idx_ref, w_ref.float()))
    m_same, m_32 = O.error_metrics(y, ref), O.error_metrics(y, ref32)
    print(f"\nE={E} dim={dim} T={tokens}: vs bf16 dataflow {m_same}\n   vs fp32 dataflow {m_32}")
    assert m_same["rel_rms"] <= 4e-3 and m_same["max_over_max"] <= 1e-2
    assert m_32["rel_rms"] <= 1e-2 and m_32["max_over_max"] <= 1e-2
    # single feed-forward through its module
    ff = m.shared_experts(x.to(dev)).cpu()
    d = O.error_metrics(ff, O.gelu_feed_forward(x, params["shared"]))
    assert d["rel_rms"] <= 4e-3, d


def test_training_mode_and_cpu_are_refused(dev):
    from comfyui_amd import hunyuan3d as H
    m = H.MoEBlock(256, num_experts=8, ff_inner_dim=1024, dtype=BF16, device=dev)
    with pytest.raises(NotImplementedError):
        m.train()(torch.zeros((1, 4, 256), dtype=BF16, device=dev))
    with pytest.raises(RuntimeError):
        m.eval()(torch.zeros((1, 4, 256), dtype=BF16))
