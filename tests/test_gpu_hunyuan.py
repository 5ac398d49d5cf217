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
@pytest.mark.parametrize("rows,K,N,bias", [(1, 256, 256, True), (300, 512, 768, True), (1025, 2048, 512, False),
                                          (10000, 256, 2048, True)])   # the last: 320-token tiles, partial last tile
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


def test_gelu_kernel(dev):
    from comfyui_amd import functional as HF
    # every finite bf16 value (65280 patterns, a multiple of 8). For |x| <= 4: equal to torch's F.gelu on the CPU or
    # one step of bf16 beside it where the two erff implementations differ in the last place. Below that 1 + erf(.)
    # cancels in fp32 and the results (of size 1e-5 and less) agree in absolute terms only; so do results in the
    # subnormal range, which torch's CPU kernel flushes to zero and the device keeps.
    bits = torch.arange(0, 65536, dtype=torch.int32)
    bits = bits[(bits & 0x7F80) != 0x7F80].to(torch.int16)
    x = bits.view(BF16)
    got = HF.gelu(x.to(dev)).cpu()
    want = torch.nn.functional.gelu(x)
    core = (x.float().abs() <= 4) & ((x.float().abs() >= 2.0 ** -120) | (x.float() == 0))
    steps = bf16_steps(got[core], want[core])
    print(f"\ngelu: max steps {int(steps.max())}, exact {(steps == 0).float().mean().item():.5f}")
    assert int(steps.max()) <= 1 and (steps == 0).float().mean().item() >= 0.98
    err = (got.float() - want.float()).abs()
    assert bool((err <= 2e-6 + 2.0 ** -7 * want.float().abs()).all()), float(err.max())
    with pytest.raises(Exception):
        HF.gelu(x[:7].to(dev))


@pytest.mark.parametrize("kind", ["fp8mm", "fp8mm_noscale", "upcast", "manual_cast"])
def test_moe_block_through_operation_classes(dev, kind):
    """MoEBlock built with one of the operation classes (hunyuandit.py:117-129 passes `operations` down to every
    Linear): the experts run one at a time through the Linear modules' own forward."""
    from comfyui_amd import hunyuan3d as H, ops, synth
    FP8 = torch.float8_e4m3fn
    E, dim, inner, tokens = 6, 256, 1024, 333
    sd, g = make_block(dim, inner, E, seed=123, bias_scale=0.2)
    x = torch.randn((1, tokens, dim), generator=g).to(BF16)
    if kind == "manual_cast":
        cls = ops.manual_cast
        m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, operations=cls, dtype=BF16, device="cpu").eval()
        m.load_state_dict(sd, strict=True)
        m.gate.to(dev)                                     # Linear weights stay on the host: cast per call
        params = O.hunyuan_params(sd, E)
    else:
        mm = kind.startswith("fp8mm")
        with_in = kind == "fp8mm"
        cls = ops.scaled_fp8_ops(fp8_matrix_mult=mm, scale_input=with_in, override_dtype=FP8)
        m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, operations=cls, dtype=BF16, device=dev).eval()
        mode = "fp8mm" if mm else "upcast"

        def quantised(prefix, s_in):
            w8, sw = synth.quantize_per_tensor(sd[prefix + "weight"].float())
            bias = sd[prefix + "bias"].to(FP8).to(BF16)    # the class keeps every parameter in the override dtype
            return O.LinearParams(w8, sw, torch.tensor(s_in) if with_in else None, bias)

        def load(ffm, prefix, s_in):
            out = []
            for lin, key in ((ffm.net[0].proj, "net.0.proj."), (ffm.net[2], "net.2.")):
                p = quantised(prefix + key, s_in)
                lin.weight = torch.nn.Parameter(p.weight.to(dev), requires_grad=False)
                with torch.no_grad():
                    lin.bias.copy_(p.bias)
                    lin.scale_weight.copy_(p.scale_weight)
                    if with_in:
                        lin.scale_input.fill_(s_in)
                out.append(p)
            return (out[0], out[1], mode)

        params = dict(gate=sd["gate.weight"], experts=[load(m.experts[i], f"experts.{i}.", 1.0 + 0.25 * i) for i in range(E)],
                      shared=load(m.shared_experts, "shared_experts.", 0.75))
        with torch.no_grad():
            m.gate.weight.copy_(sd["gate.weight"])
    assert not m.shared_experts.fusable(x.to(dev).reshape(-1, dim))
    y = m(x.to(dev)).cpu()
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    ref = O.hunyuan_moe_block(x, params, gate_result=(idx_ref, w_ref))
    d = O.error_metrics(y, ref)
    print(f"\n{kind}: {d}")
    assert d["rel_rms"] <= 1e-2 and d["max_over_max"] <= 2e-2, d
    ff = m.experts[1](x.to(dev)).cpu()
    d = O.error_metrics(ff, O.gelu_feed_forward(x, params["experts"][1]))
    assert d["rel_rms"] <= 1e-2, d


def test_training_mode_and_cpu_are_refused(dev):
    from comfyui_amd import hunyuan3d as H
    m = H.MoEBlock(256, num_experts=8, ff_inner_dim=1024, dtype=BF16, device=dev)
    with pytest.raises(NotImplementedError):
        m.train()(torch.zeros((1, 4, 256), dtype=BF16, device=dev))
    with pytest.raises(RuntimeError):
        m.eval()(torch.zeros((1, 4, 256), dtype=BF16))


def test_grouped_linear_on_320_token_tiles(dev):
    """Segment sizes at which the launcher takes the 320-token tile (232 tiles in one round instead of 288 in two):
    ragged segments, an empty expert, partial last tiles, a static group."""
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(11)
    K, N, E = 256, 2048, 7
    counts = [1500, 0, 1280, 1300, 1290, 1310, 1060]
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
            close_bf16(out[lo:hi].cpu(), torch.nn.functional.gelu(O.linear_bias(a[lo:hi], *ws[e])), frac_exact=0.93)
    close_bf16(out_sh.cpu(), torch.nn.functional.gelu(O.linear_bias(xs, *wsh)), frac_exact=0.93)
