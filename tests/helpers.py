"""Shared by the parity tests: small synthetic layers and oracle parameter packing."""
import torch

from comfyui_amd import synth
from oracle import hidream_moe_oracle as O


oracle_params = O.oracle_params


def small_layer(seed, dim, tokens, weights, num_experts=4, hidden_arg=None, scale_in=None, batch=1):
    """A small layer: returns (state_dict on CPU, x bf16 [batch, tokens/batch, dim])."""
    master, g = synth.make_weights(seed, dim=dim, hidden_arg=hidden_arg, num_experts=num_experts)
    sd = synth.to_state_dict(master, weights)
    if scale_in is not None:
        for k in list(sd):
            if k.endswith("scale_input"):
                sd[k] = torch.tensor(float(scale_in[k] if isinstance(scale_in, dict) else scale_in), dtype=torch.float32)
    x = synth.make_input(g, tokens, dim=dim, batch=batch)
    return sd, x


def set_form(name, value):
    """Switch a kernel form of the library (hdmoe_set_kernel_form). name: "HDMOE_LIGHT" or "HDMOE_SWIGLU4W";
    value: "0" = never, "1" = always, None = the launcher's own rule."""
    from comfyui_amd import _lib
    which = {"HDMOE_SWIGLU4W": _lib.FORM_SWIGLU4W, "HDMOE_LIGHT": _lib.FORM_LIGHT}[name]
    _lib.set_kernel_form(which, _lib.FORM_AUTO if value is None else (_lib.FORM_NEVER if value == "0" else _lib.FORM_ALWAYS))


def saved_forms():
    """Generator body of a fixture: restores both kernel-form switches after the test."""
    from comfyui_amd import _lib
    old = [_lib.lib.hdmoe_get_kernel_form(w) for w in (_lib.FORM_SWIGLU4W, _lib.FORM_LIGHT)]
    yield
    for w, v in zip((_lib.FORM_SWIGLU4W, _lib.FORM_LIGHT), old):
        _lib.set_kernel_form(w, v)
