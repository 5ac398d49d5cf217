"""Scaled-fp8 checkpoint ingestion for the MoE feed-forward layers: the marker tensor, the per-Linear scale
keys and the layer shapes are read straight from a state dict or a .safetensors file and the layers are built
with the matching operations class.

Follows the reference's conventions:
  * `<prefix>scaled_fp8` marker (comfy/model_detection.py:693-702): its dtype is the storage dtype of the Linear
    weights (a float32 marker means float8_e4m3fn); a marker with exactly two elements switches the fp8
    optimisations (fp8 matrix multiply, `scale_input`) off, any other size switches them on. The key is removed.
  * on saving, a scaled model carries an empty marker of its storage dtype (comfy/model_base.py:326-327).
  * Linear keys `<layer>.{shared_experts,experts.N}.{w1,w2,w3}.{weight,scale_weight,scale_input}` and
    `<layer>.gate.weight` (comfy/ldm/hidream/model.py:233-235, 255, 297-304).
  * files are opened with safetensors' own reader, tensor by tensor, onto the target device
    (comfy/utils.py:53-66); nothing is unpickled.
"""
import re

import torch

from . import hidream
from . import ops as amd_ops

FP8 = torch.float8_e4m3fn

_GATE_KEY = re.compile(r"^(.*)\.gate\.weight$")


def read_scaled_fp8_marker(state_dict, prefix=""):
    """Pop `<prefix>scaled_fp8` and return (storage dtype or None, fp8_optimizations)."""
    key = f"{prefix}scaled_fp8"
    if key not in state_dict:
        return None, False
    marker = state_dict.pop(key)
    dtype = marker.dtype
    if dtype == torch.float32:
        dtype = FP8
    return dtype, marker.nelement() != 2


def scaled_fp8_marker(dtype=FP8, fp8_optimizations=True):
    """The marker tensor a saved scaled-fp8 model carries (empty = optimisations on, two elements = off)."""
    return torch.zeros(0 if fp8_optimizations else 2, dtype=dtype)


def find_moe_layers(keys, prefix=""):
    """Layer prefixes (without trailing dot) that hold a complete MoE feed-forward, with their shapes read from the
    key set of a state dict {key: tensor or shape tuple}: {layer: dict(dim, experts, hidden, hidden_shared)}."""
    def shape(k):
        v = keys[k]
        return tuple(v.shape) if hasattr(v, "shape") else tuple(v)

    found = {}
    for k in keys:
        m = _GATE_KEY.match(k)
        if not m or not k.startswith(prefix):
            continue
        layer = m.group(1)
        w1 = f"{layer}.experts.0.w1.weight"
        sh = f"{layer}.shared_experts.w1.weight"
        if w1 not in keys or sh not in keys:
            continue
        E, dim = shape(k)
        if any(f"{layer}.experts.{e}.{w}.weight" not in keys for e in range(E) for w in ("w1", "w2", "w3")):
            raise KeyError(f"{layer}: gate has {E} experts but not all expert weights are present")
        found[layer] = dict(dim=dim, experts=E, hidden=shape(w1)[0], hidden_shared=shape(sh)[0])
    return found


def _ffn(dim, hidden, dtype, device, operations):
    # the constructor rounds int(2*h/3) up to a multiple of 256 (model.py:225-231): 3*hidden/2 maps back to hidden
    if hidden % 256 != 0:
        raise ValueError(f"hidden width {hidden} is not a multiple of 256: not a FeedForwardSwiGLU shape")
    f = hidream.FeedForwardSwiGLU(dim, 3 * hidden // 2, dtype=dtype, device=device, operations=operations)
    assert f.w1.weight.shape[0] == hidden
    return f


def build_moe_layer(shapes, operations, dtype=torch.bfloat16, device=None, top_k=2):
    """An empty MOEFeedForwardSwiGLU with exactly the checkpoint's shapes (routed and shared widths need not be
    tied to one hidden_dim argument as in the constructor)."""
    m = hidream.MOEFeedForwardSwiGLU.__new__(hidream.MOEFeedForwardSwiGLU)
    torch.nn.Module.__init__(m)
    dim = shapes["dim"]
    m.shared_experts = _ffn(dim, shapes["hidden_shared"], dtype, device, operations)
    m.experts = torch.nn.ModuleList([_ffn(dim, shapes["hidden"], dtype, device, operations)
                                     for _ in range(shapes["experts"])])
    m.gate = hidream.MoEGate(embed_dim=dim, num_routed_experts=shapes["experts"], num_activated_experts=top_k,
                             dtype=dtype, device=device, operations=operations)
    m.num_activated_experts = top_k
    return m


def _load_into(module, layer, get, available):
    """Fill a layer's Parameters from get(key); scale_input stays at its default (1.0) when the file has none."""
    own = module.state_dict()
    missing = []
    with torch.no_grad():
        for name, dst in own.items():
            key = f"{layer}.{name}"
            if key not in available:
                if not name.endswith("scale_input"):
                    missing.append(key)
                continue
            src = get(key)
            if tuple(src.shape) != tuple(dst.shape):
                raise ValueError(f"{key}: checkpoint shape {tuple(src.shape)} != module shape {tuple(dst.shape)}")
            if src.dtype != dst.dtype and (src.dtype == FP8 or dst.dtype == FP8):
                # fp8 bytes are copied as they are; a non-fp8 weight for an fp8 Linear would need quantising first
                raise TypeError(f"{key}: checkpoint dtype {src.dtype} does not match the Linear's storage dtype {dst.dtype}")
            dst.copy_(src)
    if missing:
        raise KeyError(f"missing keys: {missing}")


def load_moe_layers(source, prefix="", device=None, compute_dtype=torch.bfloat16, layers=None,
                    fast_fp8_matrix_mult=False):
    """Build every MoE feed-forward found under `prefix` in `source` (a .safetensors path or a state dict) on
    `device`. Returns ({layer prefix: module}, info) with info = dict(scaled_fp8=dtype or None,
    fp8_optimizations=bool, operations=class, shapes={layer: ...})."""
    device = torch.device(device) if device is not None else torch.device("cpu")
    if isinstance(source, dict):
        sd = dict(source)
        scaled_fp8, fp8_opt = read_scaled_fp8_marker(sd, prefix)
        shapes = find_moe_layers(sd, prefix)
        get, available, closer = (lambda k: sd[k]), sd, None
    else:
        import safetensors
        f = safetensors.safe_open(source, framework="pt", device=str(device))
        names = set(f.keys())
        marker = {}
        if f"{prefix}scaled_fp8" in names:
            marker[f"{prefix}scaled_fp8"] = f.get_tensor(f"{prefix}scaled_fp8")
        scaled_fp8, fp8_opt = read_scaled_fp8_marker(marker, prefix)
        shapes = find_moe_layers({k: f.get_slice(k).get_shape() for k in names
                                  if k.endswith(".weight") and k.startswith(prefix)}, prefix)
        get, available, closer = f.get_tensor, names, f
    try:
        weight_dtype = scaled_fp8
        if weight_dtype is None and shapes:
            first = next(iter(shapes))
            weight_dtype = get(f"{first}.experts.0.w1.weight").dtype
        operations = amd_ops.pick_operations(weight_dtype, compute_dtype, load_device=device if device.type == "cuda" else None,
                                             fp8_optimizations=fp8_opt, scaled_fp8=scaled_fp8,
                                             fast_fp8_matrix_mult=fast_fp8_matrix_mult)
        modules = {}
        for layer, shp in shapes.items():
            if layers is not None and layer not in layers:
                continue
            # non-fp8 Parameters (gate, bf16 Linears) are created in the dtype the file stores
            param_dtype = get(f"{layer}.gate.weight").dtype
            m = build_moe_layer(shp, operations, dtype=param_dtype, device=device)
            _load_into(m, layer, get, available)
            modules[layer] = m.eval()
    finally:
        if closer is not None and hasattr(closer, "__exit__"):
            closer.__exit__(None, None, None)
    return modules, dict(scaled_fp8=scaled_fp8, fp8_optimizations=fp8_opt, operations=operations, shapes=shapes)


def save_moe_layers(modules, path, prefix="", scaled_fp8=None, fp8_optimizations=True, metadata=None):
    """Write {layer prefix: module} to a .safetensors file with the marker a scaled model carries."""
    from safetensors.torch import save_file
    sd = {}
    for layer, m in modules.items():
        for k, v in m.state_dict().items():
            sd[f"{layer}.{k}"] = v.detach().cpu().contiguous()
    if scaled_fp8 is not None:
        sd[f"{prefix}scaled_fp8"] = scaled_fp8_marker(scaled_fp8, fp8_optimizations)
    save_file(sd, path, metadata=metadata)
    return sorted(sd)
