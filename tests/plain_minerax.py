"""A plain, slow Minerax in float64: one function a mechanism, whole sequences only, no cache and no kernels.

Written from the design's equations and shares nothing with the engine: the tests hold the engine's every way of
cutting a sequence against what these functions give for the sequence as a whole. ``weights`` maps tensor names to
float64 tensors, ``config`` is the dictionary a config.json holds.
"""

import math

import torch


def layer_norm(x, w, eps):
    mean = x.mean(-1, keepdim=True)
    var = ((x - mean) ** 2).mean(-1, keepdim=True)
    return (x - mean) / torch.sqrt(var + eps) * w


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def stretched_frequencies(rot):
    """Frequencies of the rotated pairs and the factor on cos and sin."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=torch.float64)
    freq = base ** (-2.0 * i / dims)
    scaling = rot.get("scaling")
    if not scaling:
        return freq, 1.0
    factor, original = scaling["factor"], scaling["original"]

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(scaling["fast"])), 0)
    hi = min(math.ceil(dim_of(scaling["slow"])), dims - 1)
    ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return freq / factor * ramp + freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate(x, rot, interleaved, first_position=0):
    """x ``[T, heads, width]``: the first rot.dims dimensions of every head turn by position."""
    if rot is None:
        return x
    dims = rot["dims"]
    freq, amplitude = stretched_frequencies(rot)
    positions = torch.arange(first_position, first_position + x.shape[0], dtype=torch.float64)
    angle = positions[:, None] * freq[None, :]
    cos, sin = (torch.cos(angle) * amplitude)[:, None, :], (torch.sin(angle) * amplitude)[:, None, :]
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    else:
        a, b = x[..., :dims // 2], x[..., dims // 2:dims]
        out[..., :dims // 2] = a * cos - b * sin
        out[..., dims // 2:dims] = b * cos + a * sin
    return out


def short_convolution(u, w):
    """u ``[T, C]``, w ``[C, taps]``: y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the start."""
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, u.shape[1], dtype=u.dtype), u])
    return sum(w[:, j] * padded[j:j + u.shape[0]] for j in range(taps))


def visible(T, window=None):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    mask = j <= i
    if window:
        mask = mask & (i - j < window)
    return mask


def softmax_with_sink(scores, mask, sink=None):
    """scores ``[heads, T, T]``; ``sink`` ``[heads]`` joins the denominator and nothing else."""
    scores = scores.masked_fill(~mask, -float("inf"))
    top = scores.max(-1, keepdim=True).values
    if sink is not None:
        top = torch.maximum(top, sink[:, None, None])
    e = torch.exp(scores - top)
    total = e.sum(-1, keepdim=True)
    if sink is not None:
        total = total + torch.exp(sink[:, None, None] - top)
    return e / total


def latent_attention(w, p, m, h, eps):
    T = h.shape[0]
    H, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m.get("vdim", m["dim"]), m["kv_rank"]
    q = (h @ w[p + "q"].T).view(T, H, d + r)
    down = h @ w[p + "dkv"].T
    latent = rms_norm(down[:, :rank], w[p + "dkv.norm"], eps)
    shared = rotate(down[:, rank:].view(T, 1, r), m.get("rot"), True)[:, 0]
    q_rot = rotate(q[..., d:], m.get("rot"), True)
    keys = (latent @ w[p + "uk"].T).view(T, H, d)
    values = (latent @ w[p + "uv"].T).view(T, H, e)
    scores = (torch.einsum("ihd,jhd->hij", q[..., :d], keys) + torch.einsum("ihd,jd->hij", q_rot, shared)) * m["scale"]
    window = m["mask"]["size"] if m.get("mask") else None
    weights = softmax_with_sink(scores, visible(T, window), w.get(p + "sink"))
    out = torch.einsum("hij,jhd->ihd", weights, values).reshape(T, H * e)
    if p + "g" in w:
        out = out * torch.sigmoid(h @ w[p + "g"].T)
    return out @ w[p + "o"].T


def conv_attention(w, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    q = short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])
    k = short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])
    v = short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])
    q = rms_norm(q, w[p + "q.norm"], eps).view(T, H, d)        # over the whole projection, all heads at once
    k = rms_norm(k, w[p + "k.norm"], eps).view(T, G, d)
    q, k = rotate(q, m.get("rot"), False), rotate(k, m.get("rot"), False)
    k = k.repeat_interleave(H // G, 1)
    v = v.view(T, G, e).repeat_interleave(H // G, 1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    if m.get("softcap"):
        scores = m["softcap"] * torch.tanh(scores / m["softcap"])
    window = m["mask"]["size"] if m.get("mask") else None
    weights = softmax_with_sink(scores, visible(T, window))
    return torch.einsum("hij,jhd->ihd", weights, v).reshape(T, H * e) @ w[p + "o"].T


def delta_rule_scan(q, k, v, beta, decay, state=None):
    """One head: q, k ``[T, d]``, v ``[T, e]``, beta ``[T]``, decay ``[T, d]``; returns outputs ``[T, e]`` and the state."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=torch.float64) if state is None else state.clone()
    out = []
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + k[t][:, None] * u[None, :]
        out.append(S.T @ q[t])
    return torch.stack(out), S


def gated_delta_rule(w, p, m, h, eps):
    T = h.shape[0]
    H, G, d, e = m["heads"], m.get("kv_heads", m["heads"]), m["dim"], m.get("vdim", m["dim"])
    silu = torch.nn.functional.silu
    q = silu(short_convolution(h @ w[p + "q"].T, w[p + "q.conv"])).view(T, G, d)
    k = silu(short_convolution(h @ w[p + "k"].T, w[p + "k.conv"])).view(T, G, d)
    v = silu(short_convolution(h @ w[p + "v"].T, w[p + "v.conv"])).view(T, H, e)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[p + "b"].T)
    step = torch.nn.functional.softplus(((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).view(T, H, d))
    decay = torch.exp(-torch.exp(w[p + "A_log"])[None, :, None] * step)
    gate = torch.sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).view(T, H, e)
    heads = []
    for head in range(H):
        source = head // (H // G)
        o, _ = delta_rule_scan(q[:, source], k[:, source], v[:, head], beta[:, head], decay[:, head])
        heads.append(o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * w[p + "norm"] * gate[:, head])
    return torch.cat(heads, dim=-1) @ w[p + "o"].T


def mixer(w, i, layer, h, eps):
    p = f"l{i}.mix."
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        return latent_attention(w, p, m, h, eps)
    return m.get("left_scale", 1.0) * conv_attention(w, p + "left.", m["left"], h, eps) + \
        m.get("right_scale", 1.0) * gated_delta_rule(w, p + "right.", m["right"], h, eps)


def feed_forward(w, i, h):
    p = f"l{i}.mlp."
    return (gelu_tanh(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def forward(config, w, tokens):
    """Logits ``[T, vocab]`` and the residual (the sum of the streams) behind every layer ``[layers, T, width]``."""
    eps = config["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)]
    count = config.get("streams")
    streams = [x.clone() for _ in range(count)] if count else None
    behind = []
    for i, layer in enumerate(config["layers"]):
        subs = [(1, lambda h: mixer(w, i, layer, h, eps))]
        if layer.get("mlp"):
            subs.append((2, lambda h: feed_forward(w, i, h)))
        for number, run in subs:
            norm_w = w[f"l{i}.norm{number}"]
            if streams is None:
                x = x + run(layer_norm(x, norm_w, eps))
                continue
            hc = f"l{i}.hc{number}."
            u = sum(w[hc + "in"][s] * streams[s] for s in range(count))
            y = run(layer_norm(u, norm_w, eps))
            streams = [sum(w[hc + "mix"][s, t] * streams[s] for s in range(count)) + w[hc + "out"][t] * y
                       for t in range(count)]
        behind.append(sum(streams) if streams is not None else x)
    logits = layer_norm(behind[-1], w["final.norm"], eps) @ w["head"].T * config.get("logit_scale", 1.0)
    return logits, torch.stack(behind)
