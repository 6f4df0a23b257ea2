"""Small Zovudra configurations for tests, and model folders made from them.

A (pages of 4): a per-token side input of 8, an embedding scale, attention with grouped heads, a rotation of part of
a head with stretched long wavelengths, a window of 9 (no multiple of the page) beside 3 kept first positions, a
routed feed-forward with four groups of which two stay, top 3, and a shared expert wider than the routed ones (two
pieces); a latent attention whose cached head (28 + 8) is padded to 48; an attention without any mask and without a
feed-forward; an attention with six query heads on one key/value head, values twice as wide as keys, a window equal to
the kept positions, experts without groups or a shared expert, top 1. B (pages of 16): no side input and no embedding
scale, twenty latent heads, a window of 40 with one kept position, groups of two experts with one group kept, a shared
expert narrower than the routed ones, more kept positions than the window is long. C (pages of 8): sizes in no step
of 8, odd head sizes, five experts. D: a window of one position beside two kept ones, twenty query heads on one
key/value head, a single expert. E: heads of 128 and a cached latent head of 128, the sizes the matrix-core kernels take.
"""

import json
import os

import torch


def _rot(dims, base, scaling=None):
    rot = {"dims": dims, "base": base}
    if scaling:
        rot["scaling"] = dict(zip(("factor", "low", "high", "original"), scaling))
    return rot


def _attention(heads, kv_heads, dim, vdim, scale, window, keep, rot):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if window:
        mixer["mask"] = {"size": window, "keep_first": keep} if keep is not None else {"size": window}
    if rot:
        mixer["rot"] = rot
    return {"type": "attention", "mixer": mixer}


def _latent(heads, dim, rot_dim, vdim, rank, q_rank, scale, window, rot):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank, "q_rank": q_rank,
             "scale": scale, "rot": rot}
    if window:
        mixer["mask"] = {"size": window}
    return {"type": "latent_attention", "mixer": mixer}


def _moe(ff, experts, top, scale=None, groups=None, shared=None):
    router = {"experts": experts, "top": top}
    if scale is not None:
        router["scale"] = scale
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": router}
    if shared:
        mlp["shared"] = {"ff": shared}
    return mlp


def _dense(ff):
    return {"kind": "dense", "ff": ff}


A = {
    "architecture": "Zovudra", "vocab": 101, "width": 64, "norm": {"eps": 1e-5}, "embedding": {"scale": 2.0},
    "token_side": {"dim": 8},
    "layers": [
        {**_attention(4, 2, 16, 16, 0.3, 9, 3, _rot(8, 100.0, (4.0, 2.0, 8.0, 64))),
         "mlp": _moe(24, 8, 3, 1.7, (4, 2), 40)},
        {**_latent(3, 24, 8, 40, 28, 20, 0.2, 5, _rot(8, 1000.0)), "mlp": _dense(40)},
        {**_attention(2, 2, 32, 32, 0.2, None, None, _rot(32, 300.0)), "mlp": None},
        {**_attention(6, 1, 16, 32, 0.25, 16, 16, _rot(16, 50.0, (2.0, 1.0, 3.0, 24))), "mlp": _moe(16, 4, 1)},
    ],
}
B = {
    "architecture": "Zovudra", "vocab": 211, "width": 96, "norm": {"eps": 1e-6},
    "layers": [
        {**_latent(20, 16, 16, 8, 48, 32, 0.15, 33, _rot(16, 777.0, (3.0, 1.0, 6.0, 32))), "mlp": _dense(72)},
        {**_attention(8, 2, 64, 64, 0.12, 40, 1, _rot(64, 5000.0, (8.0, 1.0, 4.0, 64))),
         "mlp": _moe(32, 6, 2, 0.5, (3, 1), 16)},
        {**_attention(3, 3, 48, 48, 0.15, 7, 20, _rot(24, 9000.0)), "mlp": _dense(48)},
        {**_latent(4, 32, 32, 24, 64, 16, 0.1, 16, _rot(32, 250.0)), "mlp": None},
    ],
}
C = {
    "architecture": "Zovudra", "vocab": 333, "width": 100, "norm": {"eps": 1e-4}, "embedding": {"scale": 0.5},
    "token_side": {"dim": 6},
    "layers": [
        {**_latent(5, 10, 6, 7, 13, 11, 0.3, None, _rot(6, 30.0)), "mlp": _moe(9, 5, 2, 2.25, None, 5)},
        {**_attention(3, 3, 10, 7, 0.28, 11, 2, _rot(6, 70.0, (5.0, 0.5, 2.0, 16))), "mlp": _dense(50)},
    ],
}
D = {
    "architecture": "Zovudra", "vocab": 64, "width": 48, "norm": {"eps": 1e-5}, "token_side": {"dim": 16},
    "layers": [
        {**_attention(20, 1, 16, 16, 0.25, 1, 2, _rot(16, 10000.0)), "mlp": _moe(16, 1, 1, 3.0, None, 16)},
        {**_latent(2, 8, 8, 16, 24, 8, 0.4, 1, _rot(8, 50.0)), "mlp": _dense(32)},
    ],
}
E = {
    "architecture": "Zovudra", "vocab": 150, "width": 256, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.5},
    "token_side": {"dim": 32},
    "layers": [
        {**_attention(4, 2, 128, 128, 0.09, 64, 4, _rot(128, 400000.0, (6.0, 1.0, 4.0, 128))),
         "mlp": _moe(64, 8, 2, 2.0, (2, 1), 128)},
        {**_latent(4, 64, 32, 64, 96, 48, 0.1, 40, _rot(32, 10000.0)), "mlp": _dense(128)},
        {**_attention(4, 2, 128, 128, 0.09, 64, 4, _rot(128, 400000.0, (6.0, 1.0, 4.0, 128))), "mlp": _dense(96)},
    ],
}
CONFIGS = {"A": A, "B": B, "C": C, "D": D, "E": E}
BLOCK_SIZE = {"A": 4, "B": 16, "C": 8, "D": 16, "E": 16}


def make_tensors(config: dict, seed: int, dtype: str):
    """Random tensors of the design, drawn wider than the serving default so that every mechanism moves the logits:
    an embedding of the order of one (the norm's tanh bends), matrices three times as wide and the queries more (a
    softmax mostly looks at few keys, so a window that is one position off shows), a router whose scores spread."""
    from tie_amd.models.builder import expected_tensors_for_config
    from tie_amd.weights.random_init import random_tensors

    store = torch.float32 if dtype == "float32" else torch.bfloat16
    specs = expected_tensors_for_config(config)
    tensors = dict(random_tensors(specs, seed, torch.float32, vector_dtype=torch.float32))
    for name, t in tensors.items():
        if name == "embed":
            t.mul_(25.0)
        elif name.endswith(".mix.q") or name.endswith(".mix.uq") or name.endswith(".mlp.router"):
            t.mul_(9.0)
        elif name.endswith(".shared.sg"):
            t.mul_(6.0)
        elif t.dim() == 2 and name != "side.embed":
            t.mul_(3.0)
    if dtype == "bfloat16":
        # Rounding must not change who is chosen: the first channel of a routed layer's input is made the constant 1
        # (norm weight 0, bias 1) and the router's first column holds levels 1.5 apart, in an order the seed draws,
        # further apart than the rest of the (narrow) router can move a logit. The weights still follow the tokens.
        # The float32 fixtures route by the tokens alone.
        g = torch.Generator().manual_seed(seed)
        for i, layer in enumerate(config["layers"]):
            if (layer.get("mlp") or {}).get("kind") != "moe":
                continue
            router = tensors[f"l{i}.mlp.router"]
            router.div_(9.0)
            order = torch.randperm(router.shape[0], generator=g).to(torch.float32)
            router[:, 0] = 1.5 * (order - (router.shape[0] - 1) / 2.0)
            tensors[f"l{i}.norm2"][0] = 0.0
            tensors[f"l{i}.norm2.b"][0] = 1.0
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
