"""Zovudra as a ModelSpec.

A decoder whose config.json lists its layers one by one. ``x = embed[token] * scale``; a layer is
``x += mixer(norm1(x))``, then ``x += ff(norm2(x))`` where it has a feed-forward, then (where the model has a
per-token side input) ``x += RMSnorm(W_proj (gelu_tanh(W_gate x) * side_embed[token][layer's columns])) * w``. The
model's norm is Dynamic Tanh, ``tanh(alpha x) w + b`` (``dynamic_tanh``). A layer's mixer is

* ``attention``: grouped-query softmax attention, RMS norms over the whole q and the whole k projection before the
  rotation, a rotation of the first ``rot.dims`` dimensions of a head (rotate-half pairs) whose long wavelengths are
  stretched (``rope_banded``), a sliding window beside which the first ``keep_first`` positions stay visible
  (``paged_attention`` with ``keep_first``);
* ``latent_attention``: attention whose queries come through a normed latent of their own and whose keys and values
  are made from one cached latent per token with one rotated key part for all heads, interleaved rotation, a
  sliding window (``latent_attention`` with ``q_rank``).

The feed-forward is ``down(silu(gate h) * up h)`` (``swiglu``) or a routed mixture of experts without a gate,
``down_e(relu(up_e h)^2)``: sigmoid scores, groups scored by the sum of their two best, the chosen scores divided
by their sum (+ 1e-20) times a factor, and a shared expert of the same form times ``sigmoid(w_sg . h)``
(``routed_experts``). The head norms the wanted rows and multiplies by ``head``.

Tensor names: ``embed``, ``side.embed``, ``head``, ``final.norm{,.b,.alpha}``; ``l<i>.norm1{,.b,.alpha}``,
``l<i>.norm2{,.b,.alpha}``; attention ``l<i>.mix.{q,k,v,o}`` with ``.q.norm`` and ``.k.norm``; latent attention
``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,o}``; ``l<i>.mlp.{gate,up,down}`` or ``l<i>.mlp.router``,
``l<i>.mlp.e<j>.{up,down}``, ``l<i>.mlp.shared.{up,down,sg}``; ``l<i>.side.{gate,proj,norm}``.
"""

from __future__ import annotations

from ..config.registry import register_architecture
from ..config.zovudra import DenseFfConfig, RotationConfig, ZovudraConfig
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

NAME = "Zovudra"
GROUP_TOP = 2              # a group of experts scores the sum of its two best members
RENORM_EPS = 1e-20         # joins the sum the chosen scores are divided by


def _position(rotation: RotationConfig, head_dim: int, pairing: str) -> PartSpec:
    if rotation is None:
        return PartSpec("none")
    scaling = None
    if rotation.scaling is not None:
        s = rotation.scaling
        scaling = {"factor": s.factor, "low": s.low, "high": s.high, "original": s.original}
    return PartSpec("rope_banded", {"head_dim": head_dim, "theta": rotation.base, "rotary_dim": rotation.dims,
                                    "pairing": pairing, "scaling": scaling})


def build_zovudra_spec(config: ZovudraConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps
    count = len(config.layers)

    def norm(name: str) -> PartSpec:
        return PartSpec("dynamic_tanh", {"dim": width, "weight": name, "bias": name + ".b", "alpha": name + ".alpha"})

    layers = []
    for i, layer in enumerate(config.layers):
        p = f"l{i}.mix."
        m = layer.mixer
        if layer.kind == "attention":
            mixer = PartSpec("paged_attention", {
                "hidden": width, "num_heads": m.heads, "num_kv_heads": m.kv_heads, "head_dim": m.dim,
                "value_dim": m.vdim, "scale": m.scale, "window": m.window, "keep_first": m.keep_first,
                "qk_norm": {"eps": eps, "q_weight": p + "q.norm", "k_weight": p + "k.norm", "over": "projection"},
                "position": _position(m.rotation, m.dim, "rotate_half"),
                "names": {"q": p + "q", "k": p + "k", "v": p + "v", "o": p + "o"},
            })
        else:
            mixer = PartSpec("latent_attention", {
                "hidden": width, "num_heads": m.heads, "head_dim": m.dim, "rope_dim": m.rot_dim, "value_dim": m.vdim,
                "kv_rank": m.kv_rank, "q_rank": m.q_rank, "scale": m.scale, "window": m.window, "eps": eps,
                "position": _position(m.rotation, m.rot_dim, "interleaved"),
                "names": {"dq": p + "dq", "dq_norm": p + "dq.norm", "uq": p + "uq", "dkv": p + "dkv",
                          "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv", "o": p + "o"},
            })
        norms = {"pre_mixer": norm(f"l{i}.norm1")}
        feed_forward = None
        if layer.mlp is not None:
            f = f"l{i}.mlp."
            norms["pre_feed_forward"] = norm(f"l{i}.norm2")
            if isinstance(layer.mlp, DenseFfConfig):
                feed_forward = PartSpec("swiglu", {"hidden": width, "intermediate": layer.mlp.ff, "activation": "silu",
                                                   "names": {"gate": f + "gate", "up": f + "up", "down": f + "down"}})
            else:
                r = layer.mlp
                shared = None
                if r.shared_ff is not None:
                    shared = {"intermediate": r.shared_ff, "up": f + "shared.up", "down": f + "shared.down",
                              "gate_logit": f + "shared.sg"}
                feed_forward = PartSpec("routed_experts", {
                    "hidden": width, "expert_intermediate": r.ff, "experts": r.experts, "top": r.top,
                    "groups": r.groups, "keep_groups": r.keep_groups, "scoring": "sigmoid", "group_top": GROUP_TOP,
                    "renormalize": True, "renorm_eps": RENORM_EPS, "weight_scale": r.scale,
                    "expert_activation": "relu_squared", "shared": shared,
                    "names": {"router": f + "router", "correction": None, "gate": None,
                              "up": [f"{f}e{e}.up" for e in range(r.experts)],
                              "down": [f"{f}e{e}.down" for e in range(r.experts)]},
                })
        if config.token_side_dim is None:
            block = PartSpec("pre_norm")
        else:
            d = config.token_side_dim
            block = PartSpec("pre_norm_token_side", {
                "hidden": width, "dim": d, "vocab": config.vocab, "table": "side.embed", "table_columns": count * d,
                "first": i * d, "eps": eps,
                "names": {"gate": f"l{i}.side.gate", "proj": f"l{i}.side.proj", "norm": f"l{i}.side.norm"}})
        layers.append(LayerSpec(block=block, mixer=mixer, feed_forward=feed_forward, norms=norms))
    return ModelSpec(
        architecture=NAME,
        vocab_size=config.vocab,
        hidden_size=width,
        max_positions=config.max_positions,
        embedding=PartSpec("token_embedding", {"vocab": config.vocab, "hidden": width, "weight": "embed",
                                               "scale": config.embedding_scale}),
        layers=tuple(layers),
        order=tuple(LayerCall(i) for i in range(len(layers))),
        head=PartSpec("lm_head", {"vocab": config.vocab, "hidden": width, "norm": norm("final.norm"),
                                  "weight": "head", "tied_to": None}),
    )


register_architecture(NAME, ZovudraConfig.from_json, build_zovudra_spec)
