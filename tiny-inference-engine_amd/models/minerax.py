"""Minerax as a ModelSpec.

A decoder whose config.json lists its layers one by one. Norms are layer norms with a weight and no bias. With
``streams`` in the configuration the residual is several streams (``hyper_connections``); without, every layer is
the ``pre_norm`` arrangement. A layer's mixer is

* ``latent_attention``: attention whose keys and values are made from one cached latent per token and whose
  rotated key part is shared by all heads; interleaved rotation with stretched frequencies, a sliding window, a
  learned sink per head, a sigmoid gate on the heads' outputs (``latent_attention``);
* ``parallel``: two mixers side by side on the same rows, added with a factor each (``parallel``): on the left
  grouped-query softmax attention with a short convolution on q, k and v, RMS norms over the whole q and k
  projections, a rotation of the first ``rot.dims`` dimensions of a head with stretched frequencies, and capped scores
  (``paged_attention`` with ``conv`` and a norm over the projection); on the right a gated delta rule
  (``gated_delta_rule``).

The feed-forward is ``down(gelu_tanh(gate(h)) * up(h))`` (``swiglu`` with the ``gelu_tanh`` activation). The head
norms the wanted rows, multiplies by ``head`` and scales the logits.

Tensor names: ``embed``, ``head``, ``final.norm``; ``l<i>.norm1``, ``l<i>.norm2``; ``l<i>.hc<q>.{in,out,mix}``;
latent attention ``l<i>.mix.{q,dkv,dkv.norm,uk,uv,sink,g,o}``; parallel ``l<i>.mix.left.{q,k,v,o}`` with
``.q.norm``, ``.k.norm`` and ``.{q,k,v}.conv``, ``l<i>.mix.right.{q,k,v,b,a1,a2,g1,g2,o,A_log,dt_bias,norm}`` with
``.{q,k,v}.conv``; ``l<i>.mlp.{gate,up,down}``.
"""

from __future__ import annotations

from ..config.minerax import MineraxConfig, RotationConfig
from ..config.registry import register_architecture
from .spec import LayerCall, LayerSpec, ModelSpec, PartSpec

NAME = "Minerax"


def _position(rotation: RotationConfig, head_dim: int, pairing: str) -> PartSpec:
    if rotation is None:
        return PartSpec("none")
    scaling = None
    if rotation.scaling is not None:
        s = rotation.scaling
        scaling = {"factor": s.factor, "original": s.original, "fast": s.fast, "slow": s.slow}
    return PartSpec("rope_yarn", {"head_dim": head_dim, "theta": rotation.base, "rotary_dim": rotation.dims,
                                  "pairing": pairing, "scaling": scaling})


def build_minerax_spec(config: MineraxConfig) -> ModelSpec:
    width, eps = config.width, config.norm_eps

    def norm(name: str) -> PartSpec:
        return PartSpec("layer_norm", {"dim": width, "eps": eps, "weight": name})

    layers = []
    for i, layer in enumerate(config.layers):
        p = f"l{i}.mix."
        m = layer.mixer
        if layer.kind == "latent_attention":
            mixer = PartSpec("latent_attention", {
                "hidden": width, "num_heads": m.heads, "head_dim": m.dim, "rope_dim": m.rot_dim, "value_dim": m.vdim,
                "kv_rank": m.kv_rank, "scale": m.scale, "window": m.window, "sink": p + "sink", "eps": eps,
                "position": _position(m.rotation, m.rot_dim, "interleaved"),
                "names": {"q": p + "q", "dkv": p + "dkv", "dkv_norm": p + "dkv.norm", "uk": p + "uk", "uv": p + "uv",
                          "g": p + "g", "o": p + "o"},
            })
        else:
            lp, rp = p + "left.", p + "right."
            left = PartSpec("paged_attention", {
                "hidden": width, "num_heads": m.left.heads, "num_kv_heads": m.left.kv_heads, "head_dim": m.left.dim,
                "value_dim": m.left.vdim, "scale": m.left.scale, "softcap": m.left.softcap, "window": m.left.window,
                "qk_norm": {"eps": eps, "q_weight": lp + "q.norm", "k_weight": lp + "k.norm", "over": "projection"},
                "conv": {"taps": m.left.conv, "q": lp + "q.conv", "k": lp + "k.conv", "v": lp + "v.conv"},
                "position": _position(m.left.rotation, m.left.dim, "rotate_half"),
                "names": {"q": lp + "q", "k": lp + "k", "v": lp + "v", "o": lp + "o"},
            })
            right = PartSpec("gated_delta_rule", {
                "hidden": width, "heads": m.right.heads, "kv_heads": m.right.kv_heads, "key_dim": m.right.dim,
                "value_dim": m.right.vdim, "conv": m.right.conv, "eps": eps,
                "names": {**{k: rp + k for k in ("q", "k", "v", "b", "a1", "a2", "g1", "g2", "o", "A_log", "dt_bias",
                                                 "norm")},
                          "q_conv": rp + "q.conv", "k_conv": rp + "k.conv", "v_conv": rp + "v.conv"},
            })
            mixer = PartSpec("parallel", {"hidden": width,
                                          "branches": [(left, m.left_scale), (right, m.right_scale)]})
        norms = {"pre_mixer": norm(f"l{i}.norm1")}
        feed_forward = None
        if layer.mlp is not None:
            f = f"l{i}.mlp."
            feed_forward = PartSpec("swiglu", {"hidden": width, "intermediate": layer.mlp.ff, "activation": "gelu_tanh",
                                               "names": {"gate": f + "gate", "up": f + "up", "down": f + "down"}})
            norms["pre_feed_forward"] = norm(f"l{i}.norm2")
        if config.streams is None:
            block = PartSpec("pre_norm")
        else:
            hc = {"mixer": {k: f"l{i}.hc1.{k}" for k in ("in", "out", "mix")}}
            if feed_forward is not None:
                hc["feed_forward"] = {k: f"l{i}.hc2.{k}" for k in ("in", "out", "mix")}
            block = PartSpec("hyper_connections", {"streams": config.streams, "hidden": width, "names": hc})
        layers.append(LayerSpec(block=block, mixer=mixer, feed_forward=feed_forward, norms=norms))
    return ModelSpec(
        architecture=NAME,
        vocab_size=config.vocab,
        hidden_size=width,
        max_positions=config.max_positions,
        embedding=PartSpec("token_embedding", {"vocab": config.vocab, "hidden": width, "weight": "embed"}),
        layers=tuple(layers),
        order=tuple(LayerCall(i) for i in range(len(layers))),
        head=PartSpec("lm_head", {"vocab": config.vocab, "hidden": width, "norm": norm("final.norm"),
                                  "weight": "head", "tied_to": None, "logit_scale": config.logit_scale}),
    )


register_architecture(NAME, MineraxConfig.from_json, build_minerax_spec)
