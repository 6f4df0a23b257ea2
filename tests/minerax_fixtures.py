"""Small Minerax configurations for tests, and model folders made from them.

A has two residual streams, latent attention with three heads whose cached head (28 + 8) is padded to 48, a window of
9 positions (no multiple of the page size of 4), an attention whose key and value heads differ in size (16 and 32)
with two convolution taps and capped scores beside a delta rule with grouped query/key heads, and layers without a
feed-forward. B has one plain residual (no streams), twenty latent heads (more than the matrix-core decode kernel
takes), a rotation of whole heads on the left, four taps, no cap, ungrouped delta-rule heads whose keys are wider
than their values. C has one stream, sizes in no step of 8, latent attention without a window, convolutions of one
tap (no state), no stretched frequencies, no rotation on the left at all. D has four streams and only side-by-side
layers, two of them (their states share groups), and keys of 64. E is latent attention alone with a window of one
position (a token sees itself and the sink).
"""

import json
import os

import torch


def _latent(heads, dim, rot_dim, vdim, rank, scale, window, base, scaling=None):
    rot = {"dims": rot_dim, "base": base}
    if scaling:
        rot["scaling"] = scaling
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "scale": scale, "rot": rot}
    if window:
        mixer["mask"] = {"size": window}
    return mixer


A = {
    "architecture": "Minerax", "vocab": 101, "width": 64, "norm": {"eps": 1e-5}, "streams": 2, "logit_scale": 0.5,
    "layers": [
        {"type": "latent_attention",
         "mixer": _latent(3, 24, 8, 40, 28, 0.2, 9, 100.0, {"factor": 4.0, "original": 16, "fast": 8.0, "slow": 1.0}),
         "mlp": {"kind": "dense", "ff": 40}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 32, "conv": 2, "scale": 0.3, "softcap": 5.0,
                            "rot": {"dims": 8, "base": 50.0,
                                    "scaling": {"factor": 2.0, "original": 24, "fast": 4.0, "slow": 0.5}}},
                   "right": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 24, "conv": 3},
                   "left_scale": 0.7, "right_scale": 1.6},
         "mlp": None},
        {"type": "latent_attention", "mixer": _latent(2, 16, 16, 16, 32, 0.25, 5, 1000.0), "mlp": None},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 2, "dim": 32, "vdim": 32, "conv": 3, "scale": 0.2, "softcap": 30.0,
                            "rot": {"dims": 32, "base": 300.0}},
                   "right": {"heads": 2, "kv_heads": 1, "dim": 32, "vdim": 16, "conv": 2},
                   "left_scale": 1.0, "right_scale": 0.5},
         "mlp": {"kind": "dense", "ff": 24}},
    ],
}
B = {
    "architecture": "Minerax", "vocab": 211, "width": 96, "norm": {"eps": 1e-6}, "logit_scale": 2.0,
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 6, "kv_heads": 1, "dim": 32, "vdim": 32, "conv": 4, "scale": 0.17,
                            "rot": {"dims": 32, "base": 5000.0,
                                    "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}},
                   "right": {"heads": 2, "kv_heads": 2, "dim": 40, "vdim": 16, "conv": 2},
                   "left_scale": 1.3, "right_scale": 0.9},
         "mlp": {"kind": "dense", "ff": 72}},
        {"type": "latent_attention",
         "mixer": _latent(20, 16, 16, 8, 48, 0.15, 33, 777.0, {"factor": 3.0, "original": 32, "fast": 6.0, "slow": 1.5}),
         "mlp": {"kind": "dense", "ff": 48}},
        {"type": "latent_attention", "mixer": _latent(4, 32, 32, 24, 64, 0.1, 16, 250.0), "mlp": None},
    ],
}
C = {
    "architecture": "Minerax", "vocab": 333, "width": 100, "norm": {"eps": 1e-4}, "streams": 1,
    "layers": [
        {"type": "latent_attention", "mixer": _latent(5, 10, 6, 7, 13, 0.3, None, 30.0),
         "mlp": {"kind": "dense", "ff": 50}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 3, "kv_heads": 3, "dim": 12, "vdim": 12, "conv": 1, "scale": 0.28},
                   "right": {"heads": 3, "kv_heads": 1, "dim": 20, "vdim": 9, "conv": 1},
                   "left_scale": 2.0, "right_scale": 1.0},
         "mlp": {"kind": "dense", "ff": 9}},
    ],
}
D = {
    "architecture": "Minerax", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "streams": 4, "logit_scale": 0.25,
    "layers": [
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 48, "conv": 3, "scale": 0.125, "softcap": 12.0,
                            "rot": {"dims": 16, "base": 10000.0}},
                   "right": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 80, "conv": 3},
                   "left_scale": 0.5, "right_scale": 0.5},
         "mlp": {"kind": "dense", "ff": 96}},
        {"type": "parallel",
         "mixer": {"left": {"heads": 2, "kv_heads": 1, "dim": 64, "vdim": 48, "conv": 3, "scale": 0.125, "softcap": 12.0,
                            "rot": {"dims": 16, "base": 10000.0}},
                   "right": {"heads": 2, "kv_heads": 2, "dim": 64, "vdim": 80, "conv": 3},
                   "left_scale": 1.5, "right_scale": 0.75},
         "mlp": None},
    ],
}
E = {
    "architecture": "Minerax", "vocab": 90, "width": 80, "norm": {"eps": 1e-5}, "streams": 3,
    "layers": [
        {"type": "latent_attention", "mixer": _latent(2, 8, 8, 16, 24, 0.4, 1, 50.0), "mlp": {"kind": "dense", "ff": 32}},
        {"type": "latent_attention",
         "mixer": _latent(8, 48, 16, 32, 112, 0.1, 40, 9000.0, {"factor": 2.5, "original": 20, "fast": 5.0, "slow": 1.0}),
         "mlp": None},
    ],
}
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 8, "D": 16, "E": 16}


def make_tensors(config: dict, seed: int, dtype: str):
    """Random tensors of the design, drawn wider than the serving default so that every mechanism moves the logits:
    matrices three times as wide (the queries more, so that a softmax mostly looks at one key and a window that
    is one position off shows), sinks of the order of one."""
    from tie_amd.models.builder import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    store = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = expected_tensors_for_config(config)
    tensors = dict(random_tensors(specs, seed, torch.float32, vector_dtype=torch.float32))
    for name, t in tensors.items():
        if name.endswith(".mix.q") or name.endswith(".left.q"):
            t.mul_(9.0)
        elif t.dim() == 2 and name != "embed" and ".hc" not in name and not name.endswith(".conv"):
            t.mul_(3.0)
    return {n: t.to(store) for n, t in tensors.items()}


def write_model(folder, config: dict, seed: int, dtype: str) -> str:
    from tie_amd.weights.safetensors_io import write_safetensors

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(config, f)
    write_safetensors(os.path.join(folder, "model.safetensors"), list(make_tensors(config, seed, dtype).items()))
    return str(folder)


def load_plain(folder):
    from safetensors import safe_open

    weights = {}
    with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64)
    return weights
