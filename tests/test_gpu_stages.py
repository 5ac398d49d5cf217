"""GPU parity of the individual stages, through the C ABI, against the CPU oracle."""
import pytest
import torch

from oracle import hidream_moe_oracle as O

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16
FP8 = torch.float8_e4m3fn


def _hf():
    from comfyui_amd import functional as HF
    return HF


@pytest.mark.parametrize("T,D,E", [(1, 2560, 4), (7, 2560, 4), (1024, 2560, 4), (4096, 2560, 4), (333, 512, 4),
                                   (100, 2560, 8), (64, 1024, 2), (50, 264, 16)])
def test_gate_bit_exact(dev, T, D, E):
    g = torch.Generator().manual_seed(T * 31 + D + E)
    x = torch.randn((T, D), generator=g).to(BF16)
    wg = (torch.randn((E, D), generator=g) / D ** 0.5).to(BF16)
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x, wg)
    idx, w = _hf().gate_top2(x.to(dev), wg.to(dev))
    assert torch.equal(idx.cpu(), idx_ref)
    assert torch.equal(w.cpu().view(torch.int16), w_ref.view(torch.int16))


def test_gate_exact_ties_go_to_lower_index(dev):
    # identical weight rows give identical sums whatever the order: expert 1 vs 2 tie exactly
    g = torch.Generator().manual_seed(5)
    D = 2560
    x = torch.randn((257, D), generator=g).to(BF16)
    wg = (torch.randn((4, D), generator=g) / D ** 0.5).to(BF16)
    wg[2] = wg[1]
    idx, w = _hf().gate_top2(x.to(dev), wg.to(dev))
    idx = idx.cpu()
    assert not bool(((idx[:, 0] == 2) & (idx[:, 1] == 1)).any())
    assert not bool(((idx == 2).any(dim=1) & ~(idx == 1).any(dim=1)).any())
    idx_ref, w_ref, _, _ = O.gate_fixed_order(x, wg)
    assert torch.equal(idx, idx_ref)
    # all-equal logits: experts 0 and 1
    x0 = torch.zeros((3, D), dtype=BF16)
    idx0, w0 = _hf().gate_top2(x0.to(dev), wg.to(dev))
    assert idx0.cpu().tolist() == [[0, 1]] * 3
    assert w0.cpu().float().tolist() == [[0.25, 0.25]] * 3


@pytest.mark.parametrize("T,E", [(1, 4), (5, 4), (1024, 4), (1025, 4), (8192, 4), (3000, 8), (700, 16), (8191, 2),
                                 (8193, 6), (20000, 15), (32768, 4), (32769, 4), (40000, 8), (33000, 16),
                                 (131072, 4), (150001, 5)])  # above 32768 tokens: the large-chunk kernels
def test_dispatch_bit_exact(dev, T, E):
    g = torch.Generator().manual_seed(T + E)
    first = torch.randint(0, E, (T,), generator=g)
    second = (first + torch.randint(1, E, (T,), generator=g)) % E
    idx = torch.stack([first, second], dim=1).to(torch.int32)
    counts_r, offs_r, perm_r, inv_r = O.dispatch(idx, E)
    counts, offs, perm, inv = _hf().dispatch(idx.to(dev), E)
    assert torch.equal(counts.cpu(), counts_r)
    assert torch.equal(offs.cpu(), offs_r)
    assert torch.equal(perm.cpu(), perm_r)
    assert torch.equal(inv.cpu(), inv_r)


def test_dispatch_skewed_and_empty_expert(dev):
    T, E = 2048, 4
    idx = torch.zeros((T, 2), dtype=torch.int32)
    idx[:, 1] = 1
    idx[::97, 1] = 2   # expert 3 stays empty
    ref = O.dispatch(idx, E)
    got = _hf().dispatch(idx.to(dev), E)
    for a, b in zip(got, ref):
        assert torch.equal(a.cpu(), b)
    assert int(ref[0][3]) == 0


def test_quant_fp8_all_bf16_patterns(dev):
    # every bf16 bit pattern, scale 1: must equal torch's own cast bit for bit (NaN payloads aside)
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    x = bits.view(BF16).reshape(128, 512)
    one = torch.ones((), dtype=torch.float32)
    got = _hf().quant_fp8(x.to(dev), one.to(dev)).cpu().view(torch.uint8)
    want = x.to(FP8).view(torch.uint8)
    isnan = x.float().isnan()
    assert torch.equal(got[~isnan], want[~isnan])
    assert bool(((got[isnan] & 0x7f) == 0x7f).all())
    # oracle encoder agrees too
    assert torch.equal(O.e4m3fn_encode(x.float())[~isnan], want[~isnan])


@pytest.mark.parametrize("scale", [0.5, 0.0371, 3.0])
def test_quant_fp8_scaled(dev, scale):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn((64, 2560), generator=g) * 3).to(BF16)
    s = torch.tensor(scale, dtype=torch.float32)
    want = (x * (1.0 / s).to(BF16)).to(FP8).view(torch.uint8)
    got = _hf().quant_fp8(x.to(dev), s.to(dev)).cpu().view(torch.uint8)
    assert torch.equal(got, want)


def test_quant_fp8_clamp_rule(dev):
    x = torch.tensor([[1000.0, -1000.0, 448.0, 460.0, -470.0, 0.3, 1e-4, -0.0]], dtype=torch.float32).repeat(1, 64).to(BF16)
    want = torch.clamp(x, min=-448, max=448).to(FP8).view(torch.uint8)
    got = _hf().quant_fp8(x.to(dev), None).cpu().view(torch.uint8)
    assert torch.equal(got, want)


def test_quant_permute(dev):
    g = torch.Generator().manual_seed(3)
    T, D, E = 300, 512, 4
    x = torch.randn((T, D), generator=g).to(BF16)
    first = torch.randint(0, E, (T,), generator=g)
    second = (first + torch.randint(1, E, (T,), generator=g)) % E
    idx = torch.stack([first, second], dim=1).to(torch.int32)
    counts, offs, perm, inv = O.dispatch(idx, E)
    scales = [torch.tensor(v, dtype=torch.float32) for v in (1.0, 0.5, 0.25, 2.0)]
    got = _hf().quant_permute_fp8(x.to(dev), perm.to(dev), offs.to(dev), [s.to(dev) for s in scales]).cpu()
    for e in range(E):
        lo, hi = int(offs[e]), int(offs[e + 1])
        rows = x[(perm[lo:hi] // 2).long()]
        want = (rows * (1.0 / scales[e]).to(BF16)).to(FP8)
        assert torch.equal(got[lo:hi].view(torch.uint8), want.view(torch.uint8))


# the last two shapes make the launcher pick the 320-token tile for the plain fp8 kernel (fewer rounds over the CUs)
@pytest.mark.parametrize("rows,K,N", [(256, 128, 256), (1, 2560, 256), (300, 2560, 512), (513, 6912, 2560),
                                      (1000, 384, 768), (1280, 256, 16384), (1301, 384, 16384)])
def test_linear_fp8(dev, rows, K, N):
    g = torch.Generator().manual_seed(rows + K + N)
    a = torch.randn((rows, K), generator=g).to(FP8)
    w = torch.randn((N, K), generator=g).to(FP8)
    sw = torch.tensor(0.013, dtype=torch.float32)
    si = torch.tensor(0.7, dtype=torch.float32)
    got = _hf().linear(a.to(dev), w.to(dev), sw.to(dev), si.to(dev)).cpu()
    acc = (a.double() @ w.double().t())
    want = (acc * float(si * sw)).to(BF16)
    # The matrix core does not accumulate as exact fp32: observed absolute error is about 1e-5 of the
    # typical |sum| (it shows on sums that cancel to near zero). Allow one bf16 ulp plus that floor.
    diff = (got.float() - want.float()).abs()
    tol = want.float().abs() * 2 ** -7 + 1e-3 * float(acc.abs().mean()) * float(si * sw)
    assert bool((diff <= tol).all()), float((diff / tol).max())
    assert float((got.view(torch.int16) != want.view(torch.int16)).float().mean()) < 0.03


@pytest.mark.parametrize("rows,K,N", [(256, 64, 256), (77, 2560, 512), (513, 3584, 2560)])
def test_linear_bf16(dev, rows, K, N):
    g = torch.Generator().manual_seed(rows + K + N)
    a = torch.randn((rows, K), generator=g).to(BF16)
    w = (torch.randn((N, K), generator=g) * 0.05).to(BF16)
    got = _hf().linear(a.to(dev), w.to(dev)).cpu()
    want = (a.float() @ w.float().t()).to(BF16)
    diff = (got.float() - want.float()).abs()
    tol = want.float().abs() * 2 ** -7 + 1e-4
    assert bool((diff <= tol).all()), float((diff / tol).max())


def test_combine_bit_exact(dev):
    g = torch.Generator().manual_seed(11)
    T, D = 130, 2560
    y = torch.randn((2 * T, D), generator=g).to(BF16)
    w = torch.rand((T, 2), generator=g).to(BF16)
    sh = torch.randn((T, D), generator=g).to(BF16)
    inv = torch.randperm(2 * T, generator=g).to(torch.int32)
    for shared in (sh, None):
        want = O.combine_c(y, inv, w, shared)
        got = _hf().combine(y.to(dev), inv.to(dev), w.to(dev), shared.to(dev) if shared is not None else None).cpu()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    # and the C restatement equals torch's own bf16 arithmetic for the same expression
    ys = y[inv.long()].view(T, 2, D)
    tor = (ys * w.unsqueeze(-1)).sum(dim=1) + sh
    assert torch.equal(O.combine_c(y, inv, w, sh).view(torch.int16), tor.view(torch.int16))


def test_silu_mul(dev):
    g = torch.Generator().manual_seed(12)
    a = (torch.randn((64, 1024), generator=g) * 3).to(BF16)
    b = torch.randn((64, 1024), generator=g).to(BF16)
    got = _hf().silu_mul(a.to(dev), b.to(dev)).cpu()
    want = torch.nn.functional.silu(a) * b
    # silu uses the hardware reciprocal (1 ulp of fp32), so the bf16 rounding of silu(a) can land on the
    # neighbouring value when it sits on a rounding boundary; after the product that is at most 2 bf16 ulps
    diff = (got.float() - want.float()).abs()
    assert bool((diff <= want.float().abs() * 2 ** -6 + 1e-30).all())
    assert float((got.view(torch.int16) != want.view(torch.int16)).float().mean()) < 0.01


@pytest.mark.parametrize("rows,next_scale", [(300, 1.0), (333, 0.5), (64, None)])
def test_swiglu_epilogue_cast_overflows_to_nan_like_torch(dev, rows, next_scale):
    """The gate/up GEMM casts silu(w1 x) * w3 x to e4m3fn for the w2 Linear (ops.py:337-343): beyond the rounding
    midpoint above 448 the reference's cast gives NaN (no saturation), with scale_input None it clamps first.
    Integer-valued operands and power-of-two scales make the fp32 sums exact in any order, so the only freedom left
    is the last bit of silu: values agree within one e4m3 step and NaN positions agree away from the threshold."""
    from comfyui_amd import functional as HF
    D, H = 128, 256
    g = torch.Generator().manual_seed(rows)
    a = torch.randint(-3, 4, (rows, D), generator=g).float()
    w1 = torch.randint(-3, 4, (H, D), generator=g).float()
    w3 = torch.randint(-3, 4, (H, D), generator=g).float()
    one = torch.ones((), dtype=torch.float32)
    s1, s3 = torch.tensor(0.5), torch.tensor(1.0)
    sn = None if next_scale is None else torch.tensor(float(next_scale))
    one_d = one.to(dev)
    scales = dict(scale_w1=s1.to(dev), scale_w3=s3.to(dev), scale_in1=one_d, scale_in3=one_d)
    if sn is not None:
        scales["scale_in2"] = sn.to(dev)
    w1d, w3d = w1.to(FP8).to(dev), w3.to(FP8).to(dev)
    fw = HF.make_ffn_weights(w1d, w1d, w3d, scales)      # w2 is not read by this stage
    offsets = torch.tensor([0, rows], dtype=torch.int32, device=dev)
    h = HF.grouped_swiglu(a.to(FP8).to(dev), offsets, [fw], H).cpu()
    h1 = ((a @ w1.t()) * s1).to(BF16)
    h3 = ((a @ w3.t()) * s3).to(BF16)
    m = torch.nn.functional.silu(h1) * h3                  # bf16 tensors: each op rounds to bf16
    if sn is None:
        pre = torch.clamp(m, min=-448, max=448)
    else:
        pre = m * (1.0 / sn).to(BF16)
    want = pre.to(FP8)
    got_f, want_f = h.float(), want.float()
    if sn is not None:
        assert int(want_f.isnan().sum()) > 1000                        # the overflow case is exercised
    else:
        assert int((m.float().abs() > 464).sum()) > 1000               # the clamp has something to do
        assert not bool(got_f.isnan().any()) and float(got_f.abs().max()) == 448.0
    near = (pre.float().abs() > 440) & (pre.float().abs() < 490)      # one bf16 step around 464 decides NaN or 448
    assert torch.equal(got_f.isnan() & ~near, want_f.isnan() & ~near)
    ok = ~got_f.isnan() & ~want_f.isnan()
    step = torch.maximum(want_f.abs(), torch.tensor(2.0 ** -6)) * 2.0 ** -3 * 1.001   # one e4m3 step at that magnitude
    assert bool(((got_f - want_f).abs()[ok] <= step[ok]).all())
    assert float((got_f[ok] == want_f[ok]).float().mean()) > 0.99
