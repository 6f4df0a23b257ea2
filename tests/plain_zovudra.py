"""A plain, slow implementation of the Zovudra decoder in float64, one function a mechanism, for tests.

It shares nothing with the engine: it reads the configuration dictionary and a table of tensors by name and runs
whole sequences with dense masks. Notation: T tokens, positions 0 .. T - 1; a linear weight is [out, in].
"""

import math

import torch

F64 = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms_norm(x, weight, eps):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def dynamic_tanh(x, alpha, weight, bias):
    """The norm without statistics."""
    return torch.tanh(alpha * x) * weight + bias


def banded_frequencies(rot):
    """f_i = base^(-2i / dims); with ``scaling`` long wavelengths turn ``factor`` times slower, short ones as they
    are, and those between by a blend that is linear in original / wavelength."""
    dims = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    s = rot.get("scaling")
    if not s:
        return f
    out = []
    for fi in f.tolist():
        wavelength = 2.0 * math.pi / fi
        if wavelength < s["original"] / s["high"]:
            out.append(fi)
        elif wavelength > s["original"] / s["low"]:
            out.append(fi / s["factor"])
        else:
            t = (s["original"] / wavelength - s["low"]) / (s["high"] - s["low"])
            out.append((1.0 - t) * fi / s["factor"] + t * fi)
    return torch.tensor(out, dtype=F64)


def rotate(x, positions, rot, interleaved):
    """Turns the first rot.dims dimensions of every head of x [T, heads, D]; pairs (i, i + dims/2) or (2i, 2i + 1)."""
    if rot is None:
        return x
    dims = rot["dims"]
    angle = positions.to(F64)[:, None] * banded_frequencies(rot)[None, :]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    if interleaved:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = u * c - v * s
        out[..., dims // 2:dims] = v * c + u * s
    return out


def visible(T, window, keep_first=0):
    """visible[i, j]: j <= i and (i - j < window or j < keep_first); window None: every earlier key."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = (i - j < window) if window is not None else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def softmax_attention(q, k, v, scale, mask):
    """q [T, D], k [T, D], v [T, V] of one head."""
    scores = (q @ k.T) * scale
    scores = scores.masked_fill(~mask, -math.inf)
    return torch.softmax(scores, dim=-1) @ v


def attention(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    V = m.get("vdim", D)
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    q, k = rms_norm(q, w[p + "q.norm"], eps), rms_norm(k, w[p + "k.norm"], eps)       # over all heads at once
    positions = torch.arange(T)
    q = rotate(q.view(T, H, D), positions, m.get("rot"), False)
    k = rotate(k.view(T, G, D), positions, m.get("rot"), False)
    v = v.view(T, G, V)
    mask_cfg = m.get("mask") or {}
    mask = visible(T, mask_cfg.get("size"), mask_cfg.get("keep_first", 0) if mask_cfg.get("size") else 0)
    heads = [softmax_attention(q[:, a], k[:, a // (H // G)], v[:, a // (H // G)], m["scale"], mask) for a in range(H)]
    return torch.cat(heads, dim=1) @ w[p + "o"].T


def latent_attention(h, w, p, m, eps):
    T = h.shape[0]
    H, D, R, rank = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"]
    V = m.get("vdim", D)
    c_q = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (c_q @ w[p + "uq"].T).view(T, H, D + R)
    down = h @ w[p + "dkv"].T
    c = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    positions = torch.arange(T)
    shared_key = rotate(down[:, rank:].view(T, 1, R), positions, m.get("rot"), True)[:, 0]
    q_rotated = rotate(q[..., D:], positions, m.get("rot"), True)
    keys = (c @ w[p + "uk"].T).view(T, H, D)
    values = (c @ w[p + "uv"].T).view(T, H, V)
    mask = visible(T, (m.get("mask") or {}).get("size"))
    heads = []
    for a in range(H):
        qa = torch.cat([q[:, a, :D], q_rotated[:, a]], dim=1)
        ka = torch.cat([keys[:, a], shared_key], dim=1)
        heads.append(softmax_attention(qa, ka, values[:, a], m["scale"], mask))
    return torch.cat(heads, dim=1) @ w[p + "o"].T


def dense_ff(h, w, p):
    g = h @ w[p + "gate"].T
    return (g * torch.sigmoid(g) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def expert(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


ROUTE_MARGINS = None     # a list: route() then notes how far every choice was from going the other way


def route(z, r):
    """The chosen experts [T, top] and their weights from router logits z [T, E]."""
    E, top = r["experts"], r["top"]
    s = torch.sigmoid(z)
    groups = r.get("groups") or {"count": 1, "keep": 1}
    count, keep = groups["count"], groups.get("keep", groups["count"])
    per = s.view(-1, count, E // count)
    group_score = per.topk(min(2, E // count), dim=-1).values.sum(-1)
    kept = group_score.topk(keep, dim=-1).indices
    allowed = torch.zeros_like(group_score, dtype=torch.bool).scatter_(1, kept, True)
    eligible = s.masked_fill(~allowed[:, :, None].expand_as(per).reshape(-1, E), -math.inf)
    chosen = eligible.topk(top, dim=-1).indices
    if ROUTE_MARGINS is not None:
        if keep < count:
            ranked = group_score.sort(dim=-1, descending=True).values
            ROUTE_MARGINS.append(float((ranked[:, keep - 1] - ranked[:, keep]).min()))
        ranked = eligible.sort(dim=-1, descending=True).values
        if top < E and bool(torch.isfinite(ranked[:, top]).any()):
            gap = ranked[:, top - 1] - ranked[:, top]
            ROUTE_MARGINS.append(float(gap[torch.isfinite(gap)].min()))
    weights = s.gather(1, chosen)
    weights = weights / (weights.sum(-1, keepdim=True) + 1e-20) * r.get("scale", 1.0)
    return chosen, weights


def routed_ff(h, w, p, m):
    chosen, weights = route(h @ w[p + "router"].T, m["router"])
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        for e, weight in zip(chosen[t].tolist(), weights[t]):
            out[t] += weight * expert(h[t], w[f"{p}e{e}.up"], w[f"{p}e{e}.down"])
    if m.get("shared"):
        out = out + expert(h, w[p + "shared.up"], w[p + "shared.down"]) * torch.sigmoid(h @ w[p + "shared.sg"].T)
    return out


def token_side(x, tokens, w, i, dim, eps):
    e = w["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    y = (gelu_tanh(x @ w[f"l{i}.side.gate"].T) * e) @ w[f"l{i}.side.proj"].T
    return rms_norm(y, w[f"l{i}.side.norm"], eps)


def forward(config, weights, tokens):
    """Logits [T, vocab] of every position and the residual stream after every layer."""
    w = {k: v.to(F64) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x = w["embed"][tokens] * (config.get("embedding") or {}).get("scale", 1.0)
    side_dim = (config.get("token_side") or {}).get("dim")
    streams = []

    def norm(name, rows):
        return dynamic_tanh(rows, w[name + ".alpha"], w[name], w[name + ".b"])

    for i, layer in enumerate(config["layers"]):
        h = norm(f"l{i}.norm1", x)
        mixer = attention if layer["type"] == "attention" else latent_attention
        x = x + mixer(h, w, f"l{i}.mix.", layer["mixer"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm(f"l{i}.norm2", x)
            x = x + (dense_ff(h, w, f"l{i}.mlp.") if mlp["kind"] == "dense" else routed_ff(h, w, f"l{i}.mlp.", mlp))
        if side_dim:
            x = x + token_side(x, tokens, w, i, side_dim, eps)
        streams.append(x.clone())
    return norm("final.norm", x) @ w["head"].T, streams


def greedy(config, weights, prompt, count):
    tokens, out = list(prompt), []
    for _ in range(count):
        token = int(torch.argmax(forward(config, weights, tokens)[0][-1]))
        out.append(token)
        tokens.append(token)
    return out
