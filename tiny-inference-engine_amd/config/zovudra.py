"""Typed configuration of the Zovudra decoder, read from its config.json.

Zovudra lists its layers one by one; a layer names one of two mixers, that mixer's sizes and constants, and a
feed-forward (dense, a routed mixture, or none). Nothing about a layer is assumed from another layer. Keys read:

    architecture          "Zovudra"
    vocab, width          sizes of the embedding table / the residual stream
    norm.eps              the eps of the RMS norms inside the layers (the model's own norm, Dynamic Tanh, has none)
    embedding.scale       optional: factor on the embedded rows (default 1)
    token_side.dim        optional: the size of the vector every layer receives per token; absent: no such input
    max_positions         optional: the longest sequence (default 131072; the design itself has no limit)
    layers[i].type        "attention" or "latent_attention"
    layers[i].mixer       attention: heads, kv_heads (default heads), dim, vdim (default dim), scale,
                                     mask.{size, keep_first} (both optional: a sliding window, and first positions
                                     that stay visible beside it), rot.{dims, base, scaling.{factor, low, high,
                                     original}} (optional, as is its scaling)
                          latent_attention: heads, dim, rot_dim, vdim (default dim), kv_rank, q_rank, scale,
                                     mask.size (optional), rot.{dims, base, scaling} (optional)
    layers[i].mlp         null; kind "dense" with ff; or kind "moe" with expert.ff, router.{experts, top, scale
                          (default 1), groups.{count, keep} (optional)} and shared.ff (optional)
"""

from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional, Tuple

from ..errors import LoadError, UnsupportedError
from .base import ConfigReader
from .duzozen import DEFAULT_MAX_POSITIONS, _section


@dataclasses.dataclass(frozen=True)
class BandScalingConfig:
    factor: float
    low: float                    # wavelengths above original / low turn with frequency / factor
    high: float                   # wavelengths below original / high keep their frequency
    original: float


@dataclasses.dataclass(frozen=True)
class RotationConfig:
    dims: int                     # the first ``dims`` dimensions of a (rotated part of a) head rotate
    base: float
    scaling: Optional[BandScalingConfig]


@dataclasses.dataclass(frozen=True)
class AttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: Optional[int]
    keep_first: int               # positions below this stay visible beside the window
    rotation: Optional[RotationConfig]


@dataclasses.dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                      # unrotated query / key dimensions of a head
    rot_dim: int                  # rotated ones; the key's are shared by all heads
    vdim: int
    kv_rank: int                  # size of the cached latent
    q_rank: int                   # size of the queries' latent
    scale: float
    window: Optional[int]
    rotation: Optional[RotationConfig]


@dataclasses.dataclass(frozen=True)
class DenseFfConfig:
    ff: int


@dataclasses.dataclass(frozen=True)
class RoutedFfConfig:
    ff: int                       # inner size of an expert
    experts: int
    top: int
    scale: float                  # factor on the routing weights
    groups: int
    keep_groups: int
    shared_ff: Optional[int]      # inner size of the expert every token uses; None: there is none


@dataclasses.dataclass(frozen=True)
class ZovudraLayerConfig:
    kind: str                     # "attention", "latent_attention"
    mixer: Any
    mlp: Any                      # None, DenseFfConfig or RoutedFfConfig


def _positive(where: str, **values) -> None:
    for name, value in values.items():
        if not value > 0:
            raise LoadError(f"config.json: {where} {name} must be positive, got {value}")


def _rotation(r: Optional[ConfigReader], where: str, most: int) -> Optional[RotationConfig]:
    if r is None:
        return None
    dims, base = r.integer("dims", most), r.number("base")
    if dims <= 0 or dims % 2 or dims > most:
        raise LoadError(f"config.json: {where} rotates {dims} dimensions of {most}: an even number up to that is needed")
    _positive(where + " rot", base=base)
    s = _section(r, "scaling", where + " rot", required=False)
    scaling = None
    if s is not None:
        scaling = BandScalingConfig(s.number("factor"), s.number("low"), s.number("high"), s.number("original"))
        _positive(where + " rot scaling", factor=scaling.factor, low=scaling.low, high=scaling.high,
                  original=scaling.original)
        if scaling.low == scaling.high:
            raise LoadError(f"config.json: {where} rot scaling needs 'low' and 'high' to differ")
    return RotationConfig(dims, base, scaling)


def _mask(r: ConfigReader, where: str, keeps: bool) -> Tuple[Optional[int], int]:
    mask = _section(r, "mask", where, required=False)
    if mask is None:
        return None, 0
    size = mask.integer("size", None)
    keep = mask.integer("keep_first", 0) if keeps else 0
    if size is not None and size <= 0:
        raise LoadError(f"config.json: {where} mask size must be positive, got {size}")
    if keep < 0:
        raise LoadError(f"config.json: {where} mask keep_first must not be negative, got {keep}")
    return size, (keep if size is not None else 0)       # with every key visible there is nothing to keep


@dataclasses.dataclass(frozen=True)
class ZovudraConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    token_side_dim: Optional[int]
    max_positions: int
    layers: Tuple[ZovudraLayerConfig, ...]

    @staticmethod
    def _attention(r: ConfigReader, where: str) -> AttentionConfig:
        heads = r.integer("heads")
        kv_heads, dim = r.integer("kv_heads", heads), r.integer("dim")
        vdim, scale = r.integer("vdim", dim), r.number("scale")
        _positive(where, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale)
        if heads % kv_heads:
            raise LoadError(f"config.json: {where} has {heads} query heads, no multiple of {kv_heads} key/value heads")
        window, keep = _mask(r, where, True)
        rotation = _rotation(_section(r, "rot", where, required=False), where, dim)
        return AttentionConfig(heads, kv_heads, dim, vdim, scale, window, keep, rotation)

    @staticmethod
    def _latent(r: ConfigReader, where: str) -> LatentAttentionConfig:
        heads, dim, rot_dim = r.integer("heads"), r.integer("dim"), r.integer("rot_dim")
        vdim, kv_rank, q_rank = r.integer("vdim", dim), r.integer("kv_rank"), r.integer("q_rank")
        scale = r.number("scale")
        _positive(where, heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, q_rank=q_rank, scale=scale)
        rotation = _rotation(_section(r, "rot", where, required=False), where, rot_dim)
        return LatentAttentionConfig(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, _mask(r, where, False)[0],
                                     rotation)

    @staticmethod
    def _mlp(r: Optional[ConfigReader], where: str):
        if r is None:
            return None
        kind = r.string("kind")
        if kind == "dense":
            ff = r.integer("ff")
            _positive(where + " mlp", ff=ff)
            return DenseFfConfig(ff)
        if kind != "moe":
            raise UnsupportedError(f"config.json: {where} has a feed-forward of kind '{kind}' (supported: dense, moe)")
        where += " mlp"
        ff = _section(r, "expert", where).integer("ff")
        router = _section(r, "router", where)
        experts, top, scale = router.integer("experts"), router.integer("top"), router.number("scale", 1.0)
        _positive(where, ff=ff, experts=experts, top=top)
        groups_section = _section(router, "groups", where + " router", required=False)
        groups, keep = 1, 1
        if groups_section is not None:
            groups = groups_section.integer("count")
            keep = groups_section.integer("keep", groups)
            _positive(where + " router groups", count=groups, keep=keep)
        if experts % groups or keep > groups or top > keep * (experts // groups):
            raise LoadError(f"config.json: {where} has {experts} experts in {groups} groups, {keep} kept, top {top}: "
                            f"no such choice")
        shared = _section(r, "shared", where, required=False)
        shared_ff = shared.integer("ff") if shared is not None else None
        if shared_ff is not None:
            _positive(where + " shared", ff=shared_ff)
        return RoutedFfConfig(ff, experts, top, scale, groups, keep, shared_ff)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "ZovudraConfig":
        r = ConfigReader(values)
        vocab, width = r.integer("vocab"), r.integer("width")
        eps = _section(r, "norm", "the model").number("eps")
        _positive("the model", vocab=vocab, width=width, eps=eps)
        embedding = _section(r, "embedding", "the model", required=False)
        embedding_scale = embedding.number("scale", 1.0) if embedding is not None else 1.0
        side = _section(r, "token_side", "the model", required=False)
        side_dim = side.integer("dim") if side is not None else None
        if side_dim is not None:
            _positive("the model token_side", dim=side_dim)
        entries = r.raw("layers")
        if not isinstance(entries, list) or not entries:
            raise LoadError("config.json: 'layers' must be a non-empty list")
        readers = {"attention": cls._attention, "latent_attention": cls._latent}
        layers = []
        for i, entry in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(entry, Mapping):
                raise LoadError(f"config.json: {where} must be an object")
            layer = ConfigReader(entry, f"config.json {where}")
            kind = layer.string("type")
            if kind not in readers:
                raise UnsupportedError(f"config.json: {where} has a mixer of type '{kind}' "
                                       f"(supported: {', '.join(sorted(readers))})")
            mixer = readers[kind](_section(layer, "mixer", where), where)
            layers.append(ZovudraLayerConfig(kind, mixer, cls._mlp(_section(layer, "mlp", where, required=False), where)))
        max_positions = r.integer("max_positions", DEFAULT_MAX_POSITIONS)
        _positive("the model", max_positions=max_positions)
        return cls(vocab, width, eps, embedding_scale, side_dim, max_positions, tuple(layers))
