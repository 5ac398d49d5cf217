"""Stochastic rounding of a weight tensor to an fp8 storage dtype, used by the
scaled-fp8 Linear's `set_weight` when ModelPatcher merges a LoRA into fp8 weights
(reference: comfy/float.py:14-67, called from comfy/ops.py:419-426).

On a HIP device float32 / bfloat16 values going to float8_e4m3fn take the library's kernel
(hdmoe_stochastic_round_e4m3fn, uniform numbers from Philox keyed by seed and element index). Everything
else -- host tensors of an offloaded model, float8_e5m2, other source dtypes -- is weight plumbing on the
host side of the boundary and is written with torch tensor ops below. Each value is rounded to one of its two
neighbouring fp8 values, the upper one with probability equal to its fractional
position between them; like the reference the arithmetic runs in float16 and the
uniform draws come from one generator seeded per tensor and consumed slice by slice.
"""
import torch

_FORMATS = {
    torch.float8_e4m3fn: (3, 7),   # mantissa bits, exponent bias
    torch.float8_e5m2: (2, 15),
}


def _round_slice(x, dtype, generator):
    mant_bits, bias = _FORMATS[dtype]
    exp_max = (1 << (8 - 1 - mant_bits)) - 1
    xh = x.half()
    mag = xh.abs()
    # biased exponent of the fp8 binade holding |x|; 0 marks the subnormal binade
    biased = (torch.floor(torch.log2(mag)) + bias).clamp(min=0, max=exp_max)
    normal = biased != 0
    # position inside the binade in units of one fp8 step, in [0, 2^mant_bits); the noise is added at this
    # scale, in float16, as the reference does
    pos = torch.where(normal,
                      (mag / torch.exp2(biased - bias) - 1.0) * (1 << mant_bits),
                      mag / (2.0 ** (1 - bias - mant_bits)))
    pos = pos + torch.rand(pos.size(), dtype=pos.dtype, layout=pos.layout, device=pos.device, generator=generator)
    frac = pos.floor() / (1 << mant_bits)
    out = torch.where(normal, torch.exp2(biased - bias) * (1.0 + frac), (2.0 ** (1 - bias)) * frac)
    out = torch.where(mag == 0, torch.zeros_like(out), out) * torch.sign(xh)
    lim = torch.finfo(dtype)
    return out.clamp(min=lim.min, max=lim.max)


def stochastic_rounding(value, dtype, seed=0):
    if dtype in (torch.float32, torch.float16, torch.bfloat16):
        return value.to(dtype=dtype)
    if (dtype == torch.float8_e4m3fn and value.is_cuda and value.is_contiguous()
            and value.dtype in (torch.float32, torch.bfloat16)):
        from . import functional as HF
        return HF.stochastic_round_e4m3fn(value, None, seed)
    if dtype in _FORMATS:
        generator = torch.Generator(device=value.device)
        generator.manual_seed(seed)
        output = torch.empty_like(value, dtype=dtype)
        num_slices = max(1, value.numel() / (4096 * 4096))
        slice_size = max(1, round(value.shape[0] / num_slices))
        for i in range(0, value.shape[0], slice_size):
            output[i:i + slice_size].copy_(_round_slice(value[i:i + slice_size], dtype, generator))
        return output
    return value.to(dtype=dtype)
