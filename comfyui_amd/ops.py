"""Operation classes with the attribute and method contract of ComfyUI's comfy.ops,
restricted to what the HiDream MoE feed-forward uses (Linear), computing on the
MI355X through libhdmoe.

Reference (paths under /root/reference/comfy): ops.py:61-95 cast_bias_weight,
:97-100 CastWeightBiasOp, :103-115 disable_weight_init.Linear, :282-284
manual_cast.Linear, :314-358 fp8_linear, :360-377 fp8_ops, :379-428 scaled_fp8_ops,
:449-473 pick_operations; model_management.py:1055-1072 cast_to, :1353-1375
supports_fp8_compute.

What ModelPatcher relies on and is therefore kept (model_patcher.py:98-107,
151-173, 594-619, 657-722): nn.Linear parameter names (`weight`, `bias`), the class
attributes `comfy_cast_weights`, `weight_function`, `bias_function`, the optional
`scale_weight` / `scale_input` Parameters, and the by-name hooks `convert_weight` /
`set_weight`. A class from here can be handed to a model constructor as
`operations=` or installed through model_options["custom_operations"].

Every forward needs HIP tensors; a CPU tensor raises (the package has no CPU path).
"""
import contextlib
import logging

import weakref

import torch

from . import functional as HF

FP8 = torch.float8_e4m3fn
BF16 = torch.bfloat16

# Optional side stream for weight transfers (the reference's --async-offload,
# model_management.py:1005-1053). None = transfers ride the current stream.
_offload_streams = {}


def set_offload_stream(device, stream):
    """Install (or with None remove) a side stream used for weight casts to `device`.
    Keep it at the default priority."""
    if stream is None:
        _offload_streams.pop(torch.device(device), None)
    else:
        _offload_streams[torch.device(device)] = stream


def get_offload_stream(device):
    s = _offload_streams.get(torch.device(device)) if device is not None else None
    if s is not None:
        s.wait_stream(torch.cuda.current_stream(device))
    return s


def sync_stream(device, stream):
    if stream is not None:
        torch.cuda.current_stream(device).wait_stream(stream)


def cast_to(weight, dtype=None, device=None, non_blocking=False, copy=False, stream=None):
    """model_management.cast_to: dtype/device move of a weight; returns the tensor itself
    when nothing has to change and no copy was asked for."""
    ctx = stream if stream is not None else contextlib.nullcontext()
    if device is None or weight.device == device:
        if not copy and (dtype is None or weight.dtype == dtype):
            return weight
        with ctx:
            return weight.to(dtype=dtype, copy=copy)
    with ctx:
        r = torch.empty_like(weight, dtype=dtype, device=device)
        r.copy_(weight, non_blocking=non_blocking)
    return r


def cast_bias_weight(s, input=None, dtype=None, device=None, bias_dtype=None):
    """ops.cast_bias_weight: bring `s.weight` / `s.bias` to the input's dtype and device and run
    the registered weight/bias functions (LowVramPatch objects) over the copies."""
    if input is not None:
        if dtype is None:
            dtype = input.dtype
        if bias_dtype is None:
            bias_dtype = dtype
        if device is None:
            device = input.device
    offload_stream = get_offload_stream(device)
    fn_ctx = offload_stream if offload_stream is not None else contextlib.nullcontext()
    non_blocking = device is not None and torch.device(device).type == "cuda"

    bias = None
    if s.bias is not None:
        has_fn = len(getattr(s, "bias_function", ())) > 0
        bias = cast_to(s.bias, bias_dtype, device, non_blocking=non_blocking, copy=has_fn, stream=offload_stream)
        if has_fn:
            with fn_ctx:
                for f in s.bias_function:
                    bias = f(bias)

    has_fn = len(getattr(s, "weight_function", ())) > 0
    weight = cast_to(s.weight, dtype, device, non_blocking=non_blocking, copy=has_fn, stream=offload_stream)
    if has_fn:
        with fn_ctx:
            for f in s.weight_function:
                weight = f(weight)
    sync_stream(device, offload_stream)
    return weight, bias


class CastWeightBiasOp:
    comfy_cast_weights = False
    weight_function = []
    bias_function = []


_scale_cache = {}
_scale_epoch = 0


def invalidate_scale_cache():
    """Forget every cached scale_input value. Called when a Linear of this package loads a state dict or takes a new
    weight, and when a kernel reports that a cached value was stale (take_scale_check). The cache only feeds one host
    decision (do w1 and w3 of a feed-forward share their cast factor, i.e. can the fused kernels run); the kernels
    read every scale from the device and verify that decision there, so a stale entry (`p.data.copy_()` does not bump
    the version counter the cache looks at) gives NaN and a dropped cache, never a wrong number."""
    global _scale_epoch
    _scale_epoch += 1
    _scale_cache.clear()


_scale_check_words = {}


def scale_check_word(device):
    """One pinned int32 per device that the layer's casting kernel sets to 1 when the scale_input values it finds on
    the device contradict what the host asserted from its cached copies (w1 and w3 of a feed-forward must cast the
    tokens alike); that call's output is NaN. Reading it costs no synchronisation: the module looks at it at the
    start of every forward and drops the cache (take_scale_check)."""
    t = _scale_check_words.get(device)
    if t is None:
        t = torch.zeros(1, dtype=torch.int32).pin_memory()
        _scale_check_words[device] = t
    return t


def take_scale_check(device):
    """True once after a kernel has raised the device's check word; the scale cache is dropped with it."""
    t = _scale_check_words.get(device)
    if t is None or int(t[0]) == 0:
        return False
    t.zero_()
    invalidate_scale_cache()
    logging.warning("comfyui_amd: a scale_input changed in place since its value was read; the output of the last "
                    "forward that used it is NaN. Cached scale values dropped.")
    return True


def scale_value(p, use_cache=None):
    """Host value of an fp32 scalar Parameter. A host tensor is read directly (no device involved). A device tensor is
    read once per (parameter object, version, address, cache epoch), so steady-state forwards do not synchronise.
    The entry keeps a weak reference to the tensor it was read from: an id or an address alone can be reused by a
    different tensor after the first one is freed. use_cache: None = only for device tensors."""
    if not (p.is_cuda if use_cache is None else use_cache):
        return float(p.detach().float())
    key = id(p)
    hit = _scale_cache.get(key)
    if hit is not None and hit[0]() is p and hit[1] == p._version and hit[2] == p.data_ptr() and hit[4] == _scale_epoch:
        return hit[3]
    if len(_scale_cache) > 4096:
        _scale_cache.clear()
    v = float(p.detach().float().cpu())
    _scale_cache[key] = (weakref.ref(p), p._version, p.data_ptr(), v, _scale_epoch)
    return v


def _linear_bf16(input, weight, bias):
    shape = input.shape
    x2 = input.reshape(-1, shape[-1]).contiguous()
    # a bias is added to the fp32 accumulator before the one rounding to bf16, like F.linear's fused epilogue
    out = HF.linear(x2, weight.contiguous(), bias=None if bias is None else bias.contiguous())
    return out.reshape(*shape[:-1], weight.shape[0])


class disable_weight_init:
    class Linear(torch.nn.Linear, CastWeightBiasOp):
        def reset_parameters(self):
            return None

        def _load_from_state_dict(self, *args, **kwargs):
            invalidate_scale_cache()   # load_state_dict copies into the Parameters in place
            return super()._load_from_state_dict(*args, **kwargs)

        def forward_comfy_cast_weights(self, input):
            weight, bias = cast_bias_weight(self, input)
            return _linear_bf16(input, weight, bias)

        def forward(self, *args, **kwargs):
            if self.comfy_cast_weights or len(self.weight_function) > 0 or len(self.bias_function) > 0:
                return self.forward_comfy_cast_weights(*args, **kwargs)
            return _linear_bf16(args[0], self.weight, self.bias)


class manual_cast(disable_weight_init):
    class Linear(disable_weight_init.Linear):
        comfy_cast_weights = True


_ones = {}


def _one(device):
    t = _ones.get(device)
    if t is None:
        t = torch.ones((), dtype=torch.float32, device=device)
        _ones[device] = t
    return t


def fp8_linear(self, input):
    """ops.fp8_linear on the device: quantise the activations to e4m3fn, multiply on the fp8
    matrix cores with fp32 accumulation, scale by scale_input*scale_weight, round to the input
    dtype. Returns None when the weight is not float8_e4m3fn (as the reference does).
    Unlike the reference the caller's input is left untouched when scale_input is None."""
    if self.weight.dtype != FP8:
        return None
    if input.dim() not in (2, 3):
        return None
    if input.dtype != BF16:
        raise TypeError(f"fp8_linear on the HIP path takes bfloat16 activations, got {input.dtype}")
    weight, bias = cast_bias_weight(self, input, dtype=FP8, bias_dtype=input.dtype)
    dev = input.device
    scale_weight = self.scale_weight
    scale_weight = _one(dev) if scale_weight is None else scale_weight.to(dev)
    scale_input = self.scale_input
    if scale_input is not None:
        scale_input = scale_input.to(dev)
    x2 = input.reshape(-1, input.shape[-1]).contiguous()
    xq = HF.quant_fp8(x2, scale_input)
    out = HF.linear(xq, weight.contiguous(), scale_weight, scale_input,
                    bias=None if bias is None else bias.contiguous())
    return out.reshape(*input.shape[:-1], weight.shape[0])


class fp8_ops(manual_cast):
    class Linear(manual_cast.Linear):
        def reset_parameters(self):
            self.scale_weight = None
            self.scale_input = None
            return None

        def forward_comfy_cast_weights(self, input):
            if not self.training:
                # as comfy/ops.py:367-374: whatever goes wrong in the fp8 path is logged and the Linear is
                # computed in the activation dtype instead
                try:
                    out = fp8_linear(self, input)
                    if out is not None:
                        return out
                except Exception as e:
                    logging.info("Exception during fp8 op: {}".format(e))
            weight, bias = cast_bias_weight(self, input)
            return _linear_bf16(input, weight, bias)


def scaled_fp8_ops(fp8_matrix_mult=False, scale_input=False, override_dtype=None):
    """Class factory mirroring ops.scaled_fp8_ops: Linear weights are stored as `override_dtype`
    (float8_e4m3fn) with an fp32 scalar `scale_weight` and, iff `scale_input`, an fp32 scalar
    `scale_input` (else the attribute is None)."""
    logging.info("Using scaled fp8: fp8 matrix mult: {}, scale input: {}".format(fp8_matrix_mult, scale_input))

    class scaled_fp8_op(manual_cast):
        class Linear(manual_cast.Linear):
            hdmoe_fp8_matrix_mult = fp8_matrix_mult

            def __init__(self, *args, **kwargs):
                if override_dtype is not None:
                    kwargs["dtype"] = override_dtype
                super().__init__(*args, **kwargs)

            def reset_parameters(self):
                if not hasattr(self, "scale_weight"):
                    self.scale_weight = torch.nn.parameter.Parameter(
                        data=torch.ones((), device=self.weight.device, dtype=torch.float32), requires_grad=False)
                if not scale_input:
                    self.scale_input = None
                if not hasattr(self, "scale_input"):
                    self.scale_input = torch.nn.parameter.Parameter(
                        data=torch.ones((), device=self.weight.device, dtype=torch.float32), requires_grad=False)
                return None

            def forward_comfy_cast_weights(self, input):
                if fp8_matrix_mult:
                    out = fp8_linear(self, input)
                    if out is not None:
                        return out
                # no fp8 matmul (ops.py:405-410): the weight is cast to the compute dtype and
                # scale_weight is multiplied onto the smaller of weight and input
                scale = self.scale_weight.to(input.device)
                bias = None
                if (len(self.weight_function) == 0 and self.bias is None and self.weight.dtype == FP8
                        and self.weight.device == input.device):
                    weight = self.weight  # fp8 -> bf16 is exact; the scale kernel reads the fp8 bytes directly
                else:
                    weight, bias = cast_bias_weight(self, input)
                weight = weight.contiguous()
                if weight.numel() < input.numel():
                    return _linear_bf16(input, HF.scale_to_bf16(weight, scale), bias)
                if weight.dtype == FP8:
                    weight = HF.scale_to_bf16(weight, _one(input.device))
                return _linear_bf16(HF.scale_to_bf16(input.contiguous(), scale), weight, bias)

            def convert_weight(self, weight, inplace=False, **kwargs):
                s = self.scale_weight.to(device=weight.device, dtype=weight.dtype)
                if inplace:
                    weight *= s
                    return weight
                return weight * s

            def set_weight(self, weight, inplace_update=False, seed=None, return_weight=False, **kwargs):
                from .float_round import stochastic_rounding
                if (weight.is_cuda and self.weight.dtype == torch.float8_e4m3fn and weight.is_contiguous()
                        and weight.dtype in (torch.float32, torch.bfloat16)):
                    # division, float16 rounding and stochastic rounding in one kernel
                    from . import functional as HF
                    weight = HF.stochastic_round_e4m3fn(weight, self.scale_weight.to(weight.device), seed or 0)
                else:
                    weight = stochastic_rounding(weight / self.scale_weight.to(device=weight.device, dtype=weight.dtype),
                                                 self.weight.dtype, seed=seed)
                if return_weight:
                    return weight
                if inplace_update:
                    self.weight.data.copy_(weight)
                else:
                    self.weight = torch.nn.Parameter(weight, requires_grad=False)

    return scaled_fp8_op


def supports_fp8_compute(device=None):
    """model_management.supports_fp8_compute narrowed to this build's only target: true on a
    gfx950 HIP device (the reference enables fp8 ops for gfx950 with torch >= 2.7 and ROCm >= 6.4,
    model_management.py:351-353)."""
    if not torch.cuda.is_available():
        return False
    try:
        arch = torch.cuda.get_device_properties(device if device is not None else torch.cuda.current_device()).gcnArchName
    except Exception:
        return False
    return "gfx950" in arch


def pick_operations(weight_dtype, compute_dtype, load_device=None, disable_fast_fp8=False, fp8_optimizations=False,
                    scaled_fp8=None, fast_fp8_matrix_mult=False):
    """ops.pick_operations policy. `fast_fp8_matrix_mult` stands for the reference's
    `--fast fp8_matrix_mult` command-line switch (cli_args.py:142-148), which has no global here."""
    fp8_compute = supports_fp8_compute(load_device)
    if scaled_fp8 is not None:
        return scaled_fp8_ops(fp8_matrix_mult=fp8_compute and fp8_optimizations, scale_input=fp8_optimizations,
                              override_dtype=scaled_fp8)
    if fp8_compute and (fp8_optimizations or fast_fp8_matrix_mult) and not disable_fast_fp8:
        return fp8_ops
    if compute_dtype is None or weight_dtype == compute_dtype:
        return disable_weight_init
    return manual_cast
