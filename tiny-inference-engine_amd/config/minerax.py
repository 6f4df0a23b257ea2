"""Typed configuration of the Minerax decoder, read from its config.json.

Minerax lists its layers one by one; a layer names one of two mixers, that mixer's sizes and constants, and a
feed-forward (or none). Nothing about a layer is assumed from another layer. Keys read:

    architecture          "Minerax"
    vocab, width          sizes of the embedding table / the residual stream
    norm.eps              the eps of every norm
    streams               optional: the number of residual streams (hyper-connections); absent: one plain residual sum
    logit_scale           factor on the logits (default 1)
    max_positions         optional: the longest sequence (default 131072; the design itself has no limit)
    layers[i].type        "latent_attention" or "parallel"
    layers[i].mixer       latent_attention: heads, dim, rot_dim, vdim, kv_rank, scale, mask.size (optional: a sliding
                                            window), rot.{dims, base, scaling.{factor, original, fast, slow}} (optional,
                                            as is its scaling)
                          parallel: left_scale, right_scale,
                                    left.{heads, kv_heads, dim, vdim, conv, scale, softcap (optional), rot (as above,
                                          optional), mask.size (optional)},
                                    right.{heads, kv_heads, dim, vdim, conv}
    layers[i].mlp         null, or kind "dense" with ff
"""

from __future__ import annotations

import dataclasses
from typing import Any, Mapping, Optional, Tuple

from ..errors import LoadError, UnsupportedError
from .base import ConfigReader
from .duzozen import DEFAULT_MAX_POSITIONS, _section


@dataclasses.dataclass(frozen=True)
class YarnConfig:
    factor: float
    original: float               # the context length the frequencies were made for
    fast: float                   # rotations over ``original`` positions from which a frequency is left alone
    slow: float                   # ... below which it is divided by ``factor``


@dataclasses.dataclass(frozen=True)
class RotationConfig:
    dims: int                     # the first ``dims`` dimensions of a (rotated part of a) head rotate
    base: float
    scaling: Optional[YarnConfig]


@dataclasses.dataclass(frozen=True)
class LatentAttentionConfig:
    heads: int
    dim: int                      # unrotated query / key dimensions of a head
    rot_dim: int                  # rotated ones; the key's are shared by all heads
    vdim: int
    kv_rank: int                  # size of the cached latent
    scale: float
    window: Optional[int]
    rotation: Optional[RotationConfig]


@dataclasses.dataclass(frozen=True)
class ConvAttentionConfig:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                     # taps of the short convolution on q, k and v (1: none)
    scale: float
    softcap: Optional[float]
    window: Optional[int]
    rotation: Optional[RotationConfig]


@dataclasses.dataclass(frozen=True)
class DeltaRuleConfig:
    heads: int                    # value heads (and states)
    kv_heads: int                 # query / key heads
    dim: int
    vdim: int
    conv: int


@dataclasses.dataclass(frozen=True)
class ParallelMixerConfig:
    left: ConvAttentionConfig
    right: DeltaRuleConfig
    left_scale: float
    right_scale: float


@dataclasses.dataclass(frozen=True)
class DenseFfConfig:
    ff: int


@dataclasses.dataclass(frozen=True)
class MineraxLayerConfig:
    kind: str                     # "latent_attention", "parallel"
    mixer: Any
    mlp: Optional[DenseFfConfig]


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
        scaling = YarnConfig(s.number("factor"), s.number("original"), s.number("fast"), s.number("slow"))
        _positive(where + " rot scaling", factor=scaling.factor, original=scaling.original, fast=scaling.fast,
                  slow=scaling.slow)
    return RotationConfig(dims, base, scaling)


def _window(r: ConfigReader, where: str) -> Optional[int]:
    mask = _section(r, "mask", where, required=False)
    size = mask.integer("size", None) if mask is not None else None
    if size is not None and size <= 0:
        raise LoadError(f"config.json: {where} mask size must be positive, got {size}")
    return size


@dataclasses.dataclass(frozen=True)
class MineraxConfig:
    vocab: int
    width: int
    norm_eps: float
    streams: Optional[int]
    logit_scale: float
    max_positions: int
    layers: Tuple[MineraxLayerConfig, ...]

    @staticmethod
    def _latent(r: ConfigReader, where: str) -> LatentAttentionConfig:
        heads, dim, rot_dim = r.integer("heads"), r.integer("dim"), r.integer("rot_dim")
        vdim, kv_rank, scale = r.integer("vdim", dim), r.integer("kv_rank"), r.number("scale")
        _positive(where, heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, kv_rank=kv_rank, scale=scale)
        rotation = _rotation(_section(r, "rot", where, required=False), where, rot_dim)
        return LatentAttentionConfig(heads, dim, rot_dim, vdim, kv_rank, scale, _window(r, where), rotation)

    @staticmethod
    def _left(r: ConfigReader, where: str) -> ConvAttentionConfig:
        heads = r.integer("heads")
        kv_heads, dim = r.integer("kv_heads", heads), r.integer("dim")
        vdim, conv, scale = r.integer("vdim", dim), r.integer("conv", 1), r.number("scale")
        softcap = r.number("softcap", None)
        _positive(where, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, scale=scale)
        if softcap is not None:
            _positive(where, softcap=softcap)
        if heads % kv_heads:
            raise LoadError(f"config.json: {where} has {heads} query heads, no multiple of {kv_heads} key/value heads")
        rotation = _rotation(_section(r, "rot", where, required=False), where, dim)
        return ConvAttentionConfig(heads, kv_heads, dim, vdim, conv, scale, softcap, _window(r, where), rotation)

    @staticmethod
    def _right(r: ConfigReader, where: str) -> DeltaRuleConfig:
        heads = r.integer("heads")
        kv_heads, dim = r.integer("kv_heads", heads), r.integer("dim")
        vdim, conv = r.integer("vdim", dim), r.integer("conv", 1)
        _positive(where, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv)
        if heads % kv_heads:
            raise LoadError(f"config.json: {where} has {heads} value heads, no multiple of {kv_heads} query/key heads")
        return DeltaRuleConfig(heads, kv_heads, dim, vdim, conv)

    @classmethod
    def _parallel(cls, r: ConfigReader, where: str) -> ParallelMixerConfig:
        return ParallelMixerConfig(cls._left(_section(r, "left", where), where + " left"),
                                   cls._right(_section(r, "right", where), where + " right"),
                                   r.number("left_scale", 1.0), r.number("right_scale", 1.0))

    @staticmethod
    def _mlp(r: Optional[ConfigReader], where: str) -> Optional[DenseFfConfig]:
        if r is None:
            return None
        kind = r.string("kind")
        if kind != "dense":
            raise UnsupportedError(f"config.json: {where} has a feed-forward of kind '{kind}' (supported: dense)")
        ff = r.integer("ff")
        _positive(where + " mlp", ff=ff)
        return DenseFfConfig(ff)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "MineraxConfig":
        r = ConfigReader(values)
        vocab, width = r.integer("vocab"), r.integer("width")
        eps = _section(r, "norm", "the model").number("eps")
        _positive("the model", vocab=vocab, width=width, eps=eps)
        streams = r.integer("streams", None)
        if streams is not None:
            _positive("the model", streams=streams)
        logit_scale = r.number("logit_scale", 1.0)
        entries = r.raw("layers")
        if not isinstance(entries, list) or not entries:
            raise LoadError("config.json: 'layers' must be a non-empty list")
        readers = {"latent_attention": cls._latent, "parallel": cls._parallel}
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
            layers.append(MineraxLayerConfig(kind, mixer, cls._mlp(_section(layer, "mlp", where, required=False), where)))
        max_positions = r.integer("max_positions", DEFAULT_MAX_POSITIONS)
        _positive("the model", max_positions=max_positions)
        return cls(vocab, width, eps, streams, logit_scale, max_positions, tuple(layers))
