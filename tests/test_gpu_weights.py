"""GPU parity of the weight maintenance kernel (hdmoe_stochastic_round_e4m3fn) against the CPU restatement of
/root/reference/comfy/float.py:14-67 + /root/reference/comfy/ops.py:419-426: bit-exact, same Philox draws."""
import pytest
import torch

from oracle import hidream_moe_oracle as O

pytestmark = pytest.mark.gpu
FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16


def spread_values(n, seed):
    """Magnitudes over every e4m3fn binade, the subnormal range, the saturation range, plus special values."""
    g = torch.Generator().manual_seed(seed)
    mag = torch.exp2(torch.rand(n, generator=g) * 22 - 12)          # 2^-12 .. 2^10
    x = mag * torch.where(torch.rand(n, generator=g) < 0.5, -1.0, 1.0)
    special = torch.tensor([0.0, -0.0, 448.0, -448.0, 447.9, 464.0, 480.0, 65504.0, 65520.0, 1e9, float("inf"),
                            -float("inf"), float("nan"), 2.0 ** -9, 2.0 ** -10, 2.0 ** -6, 2.0 ** -24, 2.0 ** -25,
                            1.0, 1.9999, 255.99])
    x[:special.numel()] = special
    return x.float()


@pytest.mark.parametrize("n", [1, 3, 4, 5, 1023, 65536, 1000003])
def test_f32_source_bit_exact(dev, n):
    from comfyui_amd import functional as HF
    x = spread_values(max(n, 32), seed=n)[:n].contiguous()
    for seed, scale in ((0, None), (2 ** 33 + 17, torch.tensor(0.37))):
        want = O.stochastic_round_e4m3fn(x, scale, seed).view(torch.uint8)
        got = HF.stochastic_round_e4m3fn(x.to(dev), None if scale is None else scale.to(dev), seed).cpu().view(torch.uint8)
        assert torch.equal(got, want), (got != want).nonzero()[:8].flatten().tolist()


def test_bf16_source_bit_exact(dev):
    from comfyui_amd import functional as HF
    x = spread_values(200000, seed=5).to(BF16)
    scale = torch.tensor(0.0123)
    want = O.stochastic_round_e4m3fn(x, scale, 11).view(torch.uint8)
    got = HF.stochastic_round_e4m3fn(x.to(dev), scale.to(dev), 11).cpu().view(torch.uint8)
    assert torch.equal(got, want)


def test_unbiased_on_a_weight_matrix(dev):
    from comfyui_amd import functional as HF
    g = torch.Generator().manual_seed(1)
    w = (torch.randn((2048, 2560), generator=g) * 0.02)
    s = w.abs().max() / 448
    q = HF.stochastic_round_e4m3fn(w.to(dev), s.to(dev), 3)
    back = q.float().cpu() * s
    err = back - (w / s).half().float() * s
    # zero-mean rounding error: |mean| within 5 sigma of the mean of 5.2 M independent errors
    assert abs(err.mean().item()) < 5 * err.std().item() / (w.numel() ** 0.5)
    # round-to-nearest on the same data has a comparable error size but is what this must not be
    assert not torch.equal(q.cpu().view(torch.uint8), (w / s).half().to(FP8).view(torch.uint8))


def test_set_weight_on_the_device_uses_the_kernel(dev):
    from comfyui_amd import ops as amd_ops
    ops_cls = amd_ops.scaled_fp8_ops(fp8_matrix_mult=True, scale_input=True)
    lin = ops_cls.Linear(256, 128, bias=False, device=dev, dtype=FP8)
    g = torch.Generator().manual_seed(2)
    w = torch.randn((128, 256), generator=g) * 0.5
    sw = (w.abs().max() / 448).item()                      # per-tensor scale: nothing saturates
    lin.scale_weight.data.fill_(sw)
    got = lin.set_weight(w.to(dev), seed=42, return_weight=True)
    want = O.stochastic_round_e4m3fn(w, torch.tensor(sw), 42)
    assert got.dtype == FP8 and torch.equal(got.cpu().view(torch.uint8), want.view(torch.uint8))
    lin.set_weight(w.to(dev), seed=42, inplace_update=True)
    assert torch.equal(lin.weight.data.cpu().view(torch.uint8), want.view(torch.uint8))
    # convert_weight undoes the scale: the round trip is within one fp8 step of the float16-rounded value
    back = lin.convert_weight(lin.weight.data.to(torch.float32)).cpu()
    assert bool(((back - w).abs() <= w.abs() * 2.0 ** -3 + sw * 2.0 ** -9 + 1e-6).all())


def test_bad_arguments(dev):
    from comfyui_amd import functional as HF
    with pytest.raises(TypeError):
        HF.stochastic_round_e4m3fn(torch.zeros(8, dtype=torch.float16, device=dev))
    with pytest.raises(RuntimeError):
        HF.stochastic_round_e4m3fn(torch.zeros(8))
