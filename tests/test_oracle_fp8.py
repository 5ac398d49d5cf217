"""Pins the fp8 / bf16 codecs: the oracle's (C, search based), the product's (numfmt.h, bit tricks) and
torch's own casts must agree on every input that matters. Reference semantics: `tensor.to(float8_e4m3fn)`
as used by fp8_linear (/root/reference/comfy/ops.py:337-343)."""
import ctypes
import subprocess

import pytest
import torch

from oracle import hidream_moe_oracle as O

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16


@pytest.fixture(scope="module")
def numfmt(tmp_path_factory):
    d = tmp_path_factory.mktemp("numfmt")
    so = d / "libnumfmt_host.so"
    subprocess.check_call(["g++", "-O2", "-shared", "-fPIC", "-o", str(so), "tests/numfmt_host.cpp"])
    return ctypes.CDLL(str(so))


def all_bf16_as_f32():
    bits = torch.arange(65536, dtype=torch.int32).to(torch.int16)
    return bits.view(BF16).float()


def test_decode_table_closed_form_and_torch():
    tab = O.e4m3fn_decode_table()
    ref = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(FP8).float()
    nan = ref.isnan()
    assert nan.nonzero().flatten().tolist() == [0x7F, 0xFF]
    assert torch.equal(tab[~nan], ref[~nan]) and bool(tab[nan].isnan().all())
    # known answers: largest finite, smallest subnormal, smallest normal, one, minus two
    assert tab[0x7E] == 448.0 and tab[0x01] == 2.0 ** -9 and tab[0x08] == 2.0 ** -6
    assert tab[0x38] == 1.0 and tab[0xC0] == -2.0 and tab[0x00] == 0.0


def test_oracle_encode_matches_torch_on_all_bf16_and_random_fp32():
    x = all_bf16_as_f32()
    finite = ~x.isnan()
    assert torch.equal(O.e4m3fn_encode(x)[finite], x.to(FP8).view(torch.uint8)[finite])
    g = torch.Generator().manual_seed(0)
    r = torch.randn(1 << 20, generator=g) * torch.exp(torch.randn(1 << 20, generator=g) * 3)
    assert torch.equal(O.e4m3fn_encode(r), r.to(FP8).view(torch.uint8))


def test_encode_special_cases():
    x = torch.tensor([464.0, 465.0, 448.0, 480.0, 1e9, float("inf"), 2.0 ** -10, 0.00195, 2.0 ** -10 * 1.01, -464.0,
                      -466.0, 0.0, -0.0, 2.0 ** -9 * 1.5, 2.0 ** -9 * 2.5])
    got = O.e4m3fn_encode(x).tolist()
    assert got == [0x7E, 0x7F, 0x7E, 0x7F, 0x7F, 0x7F, 0x00, 0x01, 0x01, 0xFE, 0xFF, 0x00, 0x80, 0x02, 0x02]
    assert got == x.to(FP8).view(torch.uint8).tolist()


def test_product_codec_matches_torch(numfmt):
    x = all_bf16_as_f32().contiguous()
    n = x.numel()
    out8 = torch.empty(n, dtype=torch.uint8)
    numfmt.t_f32_to_e4m3fn(ctypes.c_void_p(x.data_ptr()), ctypes.c_void_p(out8.data_ptr()), ctypes.c_long(n))
    finite = ~x.isnan()
    assert torch.equal(out8[finite], x.to(FP8).view(torch.uint8)[finite])
    assert bool(((out8[~finite] & 0x7F) == 0x7F).all())
    g = torch.Generator().manual_seed(1)
    r = (torch.randn(1 << 20, generator=g) * torch.exp(torch.randn(1 << 20, generator=g) * 3)).contiguous()
    o8 = torch.empty(r.numel(), dtype=torch.uint8)
    numfmt.t_f32_to_e4m3fn(ctypes.c_void_p(r.data_ptr()), ctypes.c_void_p(o8.data_ptr()), ctypes.c_long(r.numel()))
    assert torch.equal(o8, r.to(FP8).view(torch.uint8))
    o16 = torch.empty(r.numel(), dtype=torch.int16)
    numfmt.t_f32_to_bf16(ctypes.c_void_p(r.data_ptr()), ctypes.c_void_p(o16.data_ptr()), ctypes.c_long(r.numel()))
    assert torch.equal(o16, r.to(BF16).view(torch.int16))
    # exact ties of the bf16 rounding (low half == 0x8000) go to even
    ties = ((torch.arange(1 << 16, dtype=torch.int32) << 16) | 0x8000).view(torch.float32)
    ties = ties[ties.isfinite()].contiguous()
    t16 = torch.empty(ties.numel(), dtype=torch.int16)
    numfmt.t_f32_to_bf16(ctypes.c_void_p(ties.data_ptr()), ctypes.c_void_p(t16.data_ptr()), ctypes.c_long(ties.numel()))
    assert torch.equal(t16, ties.to(BF16).view(torch.int16))
    b = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    f = torch.empty(256, dtype=torch.float32)
    numfmt.t_e4m3fn_to_f32(ctypes.c_void_p(b.data_ptr()), ctypes.c_void_p(f.data_ptr()), ctypes.c_long(256))
    ref = b.view(FP8).float()
    assert torch.equal(f[~ref.isnan()], ref[~ref.isnan()]) and bool(f[ref.isnan()].isnan().all())


def test_per_tensor_quantisation_invariants():
    g = torch.Generator().manual_seed(2)
    w = torch.randn((300, 200), generator=g) * 0.02
    w8, s = O.quantize_weight_per_tensor(w)
    assert float(s) == pytest.approx(float(w.abs().max()) / 448.0, rel=1e-6)
    assert float(w8.float().abs().max()) == 448.0            # the amax element lands on the largest code
    err = (w8.float() * s - w).abs()
    assert float((err / w.abs().clamp_min(float(s) * 2 ** -6)).max()) <= 2 ** -4 + 1e-3   # half an e4m3 ulp
