"""Writes tests/golden/moe_small.safetensors: inputs and the CPU oracle's outputs for two tiny layers
(scaled fp8 and bf16 weights; D=256, 2 routed experts of hidden 256, shared hidden 128, 48 tokens, with
exact-tie tokens). The reference holds no vectors for this path, so these come from this repo's oracle
(oracle/hidream_moe_oracle.py); they freeze its behaviour and give the GPU tests a fixed target.

  python tests/golden/make_golden.py
"""
import os
import sys

import torch
from safetensors.torch import save_file

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from comfyui_amd import synth  # noqa: E402
from oracle import hidream_moe_oracle as O  # noqa: E402

DIM, HIDDEN_ARG, E, T = 256, 384, 2, 48


def build(weights):
    master, g = synth.make_weights(123, dim=DIM, hidden_arg=HIDDEN_ARG, num_experts=E)
    master["gate.weight"][1, 8:] = master["gate.weight"][0, 8:]      # experts nearly equal: close calls
    sd = synth.to_state_dict(master, weights)
    x = synth.make_input(g, T, dim=DIM).clone()
    x[0, ::6, :8] = 0                                                # ... and exact ties on every 6th token
    out = {}
    x2 = x.reshape(-1, DIM)
    idx, w, logits, scores = O.gate_fixed_order(x2, sd["gate.weight"])
    counts, offsets, perm, inv = O.dispatch(idx, E)
    mode = "fp8mm" if weights == "fp8" else "plain"
    y = O.moe_forward(x, O.oracle_params(sd, E), mode, gate_result=(idx, w))
    for k, v in sd.items():
        out[f"{weights}.sd.{k}"] = v.view(torch.uint8) if v.dtype == torch.float8_e4m3fn else v
    out.update({f"{weights}.x": x, f"{weights}.topk_idx": idx, f"{weights}.topk_weight": w, f"{weights}.logits": logits,
                f"{weights}.scores": scores, f"{weights}.counts": counts, f"{weights}.offsets": offsets,
                f"{weights}.perm": perm, f"{weights}.inv_perm": inv, f"{weights}.y": y})
    return out


if __name__ == "__main__":
    tensors = {}
    for wt in ("fp8", "bf16"):
        tensors.update(build(wt))
    tensors = {k: v.contiguous() for k, v in tensors.items()}
    path = os.path.join(ROOT, "tests", "golden", "moe_small.safetensors")
    save_file(tensors, path)
    print(path, os.path.getsize(path), "bytes")
