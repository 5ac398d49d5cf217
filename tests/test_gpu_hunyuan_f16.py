"""GPU parity of the Hunyuan3D-2.1 MoEBlock path with fp16 tensors
(/root/reference/comfy/ldm/hunyuan3dv2_1/hunyuandit.py:8-188 at the dtype model_management.unet_dtype picks first
from /root/reference/comfy/supported_models_base.py:46 on a device with fp16 support): gate, grouped Linear with
bias and erf GELU, GELU kernel, combine and the whole block, every rounding point in fp16."""
import pytest
import torch

from oracle import hidream_moe_oracle as O
from tests.test_oracle_branch import bf16_steps as steps16     # a monotone key over the bits: any 16-bit float format
from tests.test_oracle_hunyuan import make_block

pytestmark = pytest.mark.gpu
F16 = torch.float16


def close_f16(got, ref, frac_exact=0.95, rel=1e-3):
    """Same contraction in another summation order and erff of another library: nearly all elements identical, the
    rest within a few steps of fp16 / a small fraction of the tensor's scale."""
    st = steps16(got, ref)
    err = (got.float() - ref.float()).abs()
    assert (st == 0).float().mean().item() >= frac_exact, (st == 0).float().mean().item()
    assert bool((err <= ref.float().abs() * 2.0 ** -9 + rel * ref.float().abs().mean()).all()), err.max()


@pytest.mark.parametrize("T,D,E", [(1, 256, 2), (700, 2048, 8), (333, 1024, 6), (4100, 512, 16), (65, 2560, 4)])
def test_gate_f16_bit_exact(dev, T, D, E):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(T + D + E)
    x = torch.randn((T, D), generator=g).to(F16)
    wg = (torch.randn((E, D), generator=g) / D ** 0.5).to(F16)
    if T > 64:
        x[7] = x[3]                     # identical rows route identically
        wg[1] = wg[0]                   # experts 0 and 1 tie exactly on every token: the lower index goes first
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x, wg)
    idx, w = HF.gate_top2(x.to(dev), wg.to(dev))
    assert w.dtype == F16
    assert torch.equal(idx.cpu(), idx_ref)
    assert torch.equal(w.cpu().view(torch.int16), w_ref.view(torch.int16))
    with pytest.raises(TypeError):
        HF.gate_top2(x.to(dev), wg.to(dev).to(torch.bfloat16))


@pytest.mark.parametrize("act", ["none", "gelu"])
@pytest.mark.parametrize("rows,K,N,bias", [(1, 256, 256, True), (300, 512, 768, True), (1025, 2048, 512, False),
                                          (10000, 256, 2048, True)])   # the last: 320-token tiles, partial last tile
def test_single_linear_with_bias_and_gelu_f16(dev, act, rows, K, N, bias):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(rows + K)
    x = torch.randn((rows, K), generator=g).to(F16)
    w = (torch.randn((N, K), generator=g) / K ** 0.5).to(F16)
    b = torch.randn((N,), generator=g).to(F16) if bias else None
    ref = O.linear_bias(x, w, b)
    assert ref.dtype == F16
    if act == "gelu":
        ref = torch.nn.functional.gelu(ref.float()).to(F16)
    xd = x.to(dev)
    _, got = HF.grouped_linear(xd[:0], None, [], a_static=xd, shared=(w.to(dev), None if b is None else b.to(dev)), act=act)
    assert got.dtype == F16
    close_f16(got.cpu(), ref)
    if act == "none":
        # the single-Linear entry point with the fp16 weight code
        got2 = HF.linear(xd, w.to(dev), bias=None if b is None else b.to(dev))
        assert got2.dtype == F16 and torch.equal(got2, got)


def test_linear_f16_exact_on_integers_and_overflow(dev):
    """Integer-valued operands: every product and partial sum exact, so the result is exact; sums beyond 65504
    become infinity as torch's fp16 conversion makes them."""
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(2)
    x = torch.randint(-4, 5, (130, 256), generator=g).float()
    w = torch.randint(-4, 5, (256, 256), generator=g).float()
    b = torch.randint(-8, 9, (256,), generator=g).float()
    want = (x.double() @ w.double().t() + b.double()).to(F16)
    got = HF.linear(x.to(F16).to(dev), w.to(F16).to(dev), bias=b.to(F16).to(dev)).cpu()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    xb = torch.full((2, 256), 64.0)
    wb = torch.full((256, 256), 8.0)
    got = HF.linear(xb.to(F16).to(dev), wb.to(F16).to(dev)).cpu()            # 64 * 8 * 256 = 131072 > 65504
    assert bool(torch.isinf(got).all()) and bool((got > 0).all())


def test_grouped_linear_f16_segments(dev):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(7)
    K, N, E = 256, 512, 6
    counts = [0, 37, 300, 0, 1, 257]
    rows = sum(counts)
    offsets = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
    a = torch.randn((rows, K), generator=g).to(F16)
    ws = [((torch.randn((N, K), generator=g) / 16).to(F16), torch.randn((N,), generator=g).to(F16)) for _ in range(E)]
    xs = torch.randn((90, K), generator=g).to(F16)
    wsh = ((torch.randn((N, K), generator=g) / 16).to(F16), torch.randn((N,), generator=g).to(F16))
    out, out_sh = HF.grouped_linear(a.to(dev), offsets.to(dev), [(w.to(dev), b.to(dev)) for w, b in ws],
                                    a_static=xs.to(dev), shared=(wsh[0].to(dev), wsh[1].to(dev)), act="gelu")
    gelu = lambda t: torch.nn.functional.gelu(t.float()).to(F16)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            close_f16(out[lo:hi].cpu(), gelu(O.linear_bias(a[lo:hi], *ws[e])), frac_exact=0.93)
    close_f16(out_sh.cpu(), gelu(O.linear_bias(xs, *wsh)), frac_exact=0.93)
    with pytest.raises(TypeError):      # mixed formats are refused
        HF.grouped_linear(a.to(dev), offsets.to(dev), [(w.to(dev).to(torch.bfloat16), b.to(dev)) for w, b in ws])


def test_gelu_kernel_f16(dev):
    from comfyui_amd import functional as HF
    # every finite fp16 value. For 2^-10 <= |x| and -2 <= x <= 4: torch's F.gelu (evaluated in fp32 here, rounded
    # once) or one step beside it where the two erff differ in the last place; elsewhere (1 + erf cancels in fp32
    # for x below -2, which fp16's finer steps show from there on; tiny results) agreement in absolute terms.
    bits = torch.arange(0, 65536, dtype=torch.int32)
    bits = bits[(bits & 0x7C00) != 0x7C00].to(torch.int16)
    assert bits.numel() % 8 == 0
    x = bits.view(F16)
    got = HF.gelu(x.to(dev)).cpu()
    want = torch.nn.functional.gelu(x.float()).to(F16)
    core = ((x.float() <= 4) & (x.float() >= -2) & (x.float().abs() >= 2.0 ** -10)) | (x.float() == 0)
    st = steps16(got[core], want[core])
    print(f"\ngelu f16: max steps {int(st.max())}, exact {(st == 0).float().mean().item():.5f}")
    assert int(st.max()) <= 1 and (st == 0).float().mean().item() >= 0.98
    err = (got.float() - want.float()).abs()
    assert bool((err <= 2e-6 + 2.0 ** -10 * want.float().abs()).all()), float(err.max())


def test_combine_f16_bit_exact(dev):
    """bf16 -> fp16 everywhere in the combine's formula: fp16( fp16( fp16(y0 w0) + fp16(y1 w1) ) + shared ), the
    products, the two-term sum and the last sum as torch's fp16 elementwise kernels round them."""
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(3)
    T, D, E = 517, 264, 5
    scores = torch.rand((T, E), generator=g)
    idx = torch.topk(scores, 2, dim=-1).indices.to(torch.int32)
    w = torch.rand((T, 2), generator=g).to(F16)
    _, _, perm, inv = O.dispatch(idx, E)
    y = (torch.randn((2 * T, D), generator=g) * 3).to(F16)
    sh = torch.randn((T, D), generator=g).to(F16)
    inv2 = inv.view(T, 2).long()
    a = y[inv2[:, 0]] * w[:, 0:1]
    b = y[inv2[:, 1]] * w[:, 1:2]
    want = (a + b) + sh
    got = HF.combine(y.to(dev), inv.to(dev), w.to(dev), sh.to(dev)).cpu()
    assert got.dtype == F16 and torch.equal(got.view(torch.int16), want.view(torch.int16))
    got = HF.combine(y.to(dev), inv.to(dev), w.to(dev), None).cpu()
    assert torch.equal(got.view(torch.int16), (a + b).view(torch.int16))


@pytest.mark.parametrize("E,dim,inner,tokens", [(8, 512, 2048, 700), (6, 256, 1024, 65), (8, 2048, 8192, 1500)])
def test_moe_block_f16(dev, E, dim, inner, tokens):
    from comfyui_amd import hunyuan3d as H
    sd, g = make_block(dim, inner, E, seed=E + dim, dtype=F16, bias_scale=0.2)
    x = torch.randn((1, tokens, dim), generator=g).to(F16)
    m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, dtype=F16, device=dev).eval()
    m.load_state_dict({k: v.to(dev) for k, v in sd.items()}, strict=True)
    y = m(x.to(dev)).cpu()
    assert y.shape == x.shape and y.dtype == F16
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd["gate.weight"])
    idx, w, aux = m.gate(x.to(dev))
    assert aux is None and idx.dtype == torch.int64 and w.dtype == F16
    assert torch.equal(idx.cpu(), idx_ref.long()) and torch.equal(w.cpu().view(torch.int16), w_ref.view(torch.int16))
    params = O.hunyuan_params(sd, E)
    ref = O.hunyuan_moe_block(x, params, gate_result=(idx_ref, w_ref))
    assert ref.dtype == F16
    ref32 = O.hunyuan_moe_block(x.float(), {k: ([tuple(t.float() for t in ff) for ff in v] if k == "experts"
                                                  else (v.float() if k == "gate" else tuple(t.float() for t in v)))
                                             for k, v in params.items()}, gate_result=(idx_ref, w_ref.float()))
    m_same, m_32 = O.error_metrics(y, ref), O.error_metrics(y, ref32)
    print(f"\nf16 E={E} dim={dim} T={tokens}: vs fp16 dataflow {m_same}\n   vs fp32 dataflow {m_32}")
    # fp16 carries 3 more mantissa bits than bf16: an eighth of the bf16 bounds
    assert m_same["rel_rms"] <= 5e-4 and m_same["max_over_max"] <= 1.5e-3
    assert m_32["rel_rms"] <= 1.5e-3 and m_32["max_over_max"] <= 1.5e-3
    ff = m.shared_experts(x.to(dev)).cpu()
    d = O.error_metrics(ff, O.gelu_feed_forward(x, params["shared"]))
    assert d["rel_rms"] <= 5e-4, d


def test_moe_block_f16_with_cast_weights(dev):
    """Weights stored in bf16, activations fp16, manual-cast operations (ops.py:283-284): every Linear casts its
    weight and bias to fp16 per call and the experts run one at a time."""
    from comfyui_amd import hunyuan3d as H
    from comfyui_amd import ops
    E, dim, inner, tokens = 6, 256, 1024, 300
    sd, g = make_block(dim, inner, E, seed=77, dtype=torch.bfloat16, bias_scale=0.2)
    x = torch.randn((1, tokens, dim), generator=g).to(F16)
    m = H.MoEBlock(dim, num_experts=E, moe_top_k=2, ff_inner_dim=inner, dtype=torch.bfloat16, device=dev,
                   operations=ops.manual_cast).eval()
    m.load_state_dict({k: v.to(dev) for k, v in sd.items()}, strict=True)
    y = m(x.to(dev)).cpu()
    assert y.dtype == F16
    sd16 = {k: v.to(F16) for k, v in sd.items()}
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x.reshape(-1, dim), sd16["gate.weight"])
    ref = O.hunyuan_moe_block(x, O.hunyuan_params(sd16, E), gate_result=(idx_ref, w_ref))
    d = O.error_metrics(y, ref)
    print("\nf16 manual cast", d)
    assert d["rel_rms"] <= 5e-4 and d["max_over_max"] <= 1.5e-3


def test_f32_activations_are_refused(dev):
    from comfyui_amd import hunyuan3d as H
    m = H.MoEBlock(256, num_experts=6, moe_top_k=2, ff_inner_dim=1024, dtype=torch.float32, device=dev).eval()
    with pytest.raises(RuntimeError):
        m(torch.zeros((1, 8, 256), dtype=torch.float32, device=dev))


def test_grouped_linear_on_320_token_tiles_f16(dev):
    """Segment sizes at which the launcher takes the 320-token tile (232 tiles in one round instead of 288 in two):
    ragged segments, an empty expert, partial last tiles, a static group."""
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(11)
    K, N, E = 256, 2048, 7
    counts = [1500, 0, 1280, 1300, 1290, 1310, 1060]
    rows = sum(counts)
    offsets = torch.tensor([0] + torch.tensor(counts).cumsum(0).tolist(), dtype=torch.int32)
    a = torch.randn((rows, K), generator=g).to(F16)
    ws = [((torch.randn((N, K), generator=g) / 16).to(F16), torch.randn((N,), generator=g).to(F16)) for _ in range(E)]
    xs = torch.randn((90, K), generator=g).to(F16)
    wsh = ((torch.randn((N, K), generator=g) / 16).to(F16), torch.randn((N,), generator=g).to(F16))
    out, out_sh = HF.grouped_linear(a.to(dev), offsets.to(dev), [(w.to(dev), b.to(dev)) for w, b in ws],
                                    a_static=xs.to(dev), shared=(wsh[0].to(dev), wsh[1].to(dev)), act="gelu")
    gelu = lambda t: torch.nn.functional.gelu(t.float()).to(F16)
    for e in range(E):
        lo, hi = int(offsets[e]), int(offsets[e + 1])
        if hi > lo:
            close_f16(out[lo:hi].cpu(), gelu(O.linear_bias(a[lo:hi], *ws[e])), frac_exact=0.93)
    close_f16(out_sh.cpu(), gelu(O.linear_bias(xs, *wsh)), frac_exact=0.93)
