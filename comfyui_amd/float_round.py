"""Stochastic rounding of a weight tensor to an fp8 storage dtype, used by the
scaled-fp8 Linear's `set_weight` when ModelPatcher merges a LoRA into fp8 weights
(reference: comfy/float.py:14-67, called from comfy/ops.py:419-426).

This is weight maintenance on the host side of the boundary, not part of the forward
path, and is written with torch tensor ops. Each value is rounded to one of its two
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
    xh = x.half()
    mag = xh.abs()
    # exponent of the fp8 binade that holds |x| (subnormals share the lowest one)
    expo = torch.floor(torch.log2(mag)).clamp(min=1 - bias, max=(1 << (8 - 1 - mant_bits)) - 1 - bias)
    expo = torch.where(mag == 0, torch.full_like(expo, 1 - bias), expo)
    ulp = torch.exp2(expo - mant_bits)
    steps = mag / ulp
    steps = torch.floor(steps + torch.rand(steps.size(), dtype=steps.dtype, layout=steps.layout,
                                           device=steps.device, generator=generator))
    out = torch.sign(xh) * steps * ulp
    lim = torch.finfo(dtype)
    return out.clamp(min=lim.min, max=lim.max)


def stochastic_rounding(value, dtype, seed=0):
    if dtype in (torch.float32, torch.float16, torch.bfloat16):
        return value.to(dtype=dtype)
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
