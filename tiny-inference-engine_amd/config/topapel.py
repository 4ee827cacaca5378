"""Typed configuration of the Topapel decoder, read from its config.json.

Topapel lists its layers one by one; a layer names one of three mixers, that mixer's sizes and constants, and a
feed-forward (or none). Nothing about a layer is assumed from another layer. Keys read:

    architecture          "Topapel"
    vocab, width          sizes of the embedding table / the residual stream
    embedding.scale       factor on the embedded rows (default 1)
    norm.eps              the eps of every RMS norm
    logit_scale           factor on the logits (default 1);  logit_softcap  c: logits <- c tanh(logits / c) (optional)
    max_positions         optional: the longest sequence (default 131072; the design itself has no limit)
    layers[i].type        "lightning", "attention" or "mingru"
    layers[i].mixer       lightning: heads, dim, vdim, decay (one number a head)
                          attention: heads, kv_heads, dim, vdim (= dim: the values are the keys), scale,
                                     mask.size (optional: causal chunks), rot.{dims, base, scaling.factor} (optional)
                          mingru:    width
    layers[i].mlp         null, or kind "dense" with ff
"""

from __future__ import annotations

import dataclasses
import math
from typing import Any, Mapping, Optional, Tuple

from ..errors import LoadError, UnsupportedError
from .base import ConfigReader
from .duzozen import DEFAULT_MAX_POSITIONS, _section


@dataclasses.dataclass(frozen=True)
class LightningMixerConfig:
    heads: int
    dim: int                      # size of a query / key head
    vdim: int                     # size of a value head
    decay: Tuple[float, ...]      # one factor a head


@dataclasses.dataclass(frozen=True)
class RotationConfig:
    dims: int                     # the first ``dims`` dimensions of a head rotate
    base: float
    factor: float                 # linear scaling: frequencies are divided by it


@dataclasses.dataclass(frozen=True)
class ChunkedAttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int
    scale: float
    chunk: Optional[int]          # None: plain causal attention
    rotation: Optional[RotationConfig]


@dataclasses.dataclass(frozen=True)
class MinGruMixerConfig:
    width: int


@dataclasses.dataclass(frozen=True)
class DenseFfConfig:
    ff: int


@dataclasses.dataclass(frozen=True)
class TopapelLayerConfig:
    kind: str                     # "lightning", "attention", "mingru"
    mixer: Any
    mlp: Optional[DenseFfConfig]


def _positive(where: str, **values) -> None:
    for name, value in values.items():
        if value <= 0:
            raise LoadError(f"config.json: {where} mixer {name} must be positive, got {value}")


@dataclasses.dataclass(frozen=True)
class TopapelConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    logit_softcap: Optional[float]
    max_positions: int
    layers: Tuple[TopapelLayerConfig, ...]

    @staticmethod
    def _lightning(r: ConfigReader, where: str) -> LightningMixerConfig:
        heads, dim = r.integer("heads"), r.integer("dim")
        vdim = r.integer("vdim", dim)
        _positive(where, heads=heads, dim=dim, vdim=vdim)
        decay = r.raw("decay")
        if not isinstance(decay, list) or len(decay) != heads or \
                not all(isinstance(d, (int, float)) and not isinstance(d, bool) and math.isfinite(d) for d in decay):
            raise LoadError(f"config.json: {where} mixer decay must list one number for each of the {heads} heads")
        return LightningMixerConfig(heads, dim, vdim, tuple(float(d) for d in decay))

    @staticmethod
    def _attention(r: ConfigReader, where: str) -> ChunkedAttentionMixerConfig:
        heads = r.integer("heads")
        kv_heads = r.integer("kv_heads", heads)
        dim = r.integer("dim")
        vdim = r.integer("vdim", dim)
        scale = r.number("scale")
        _positive(where, heads=heads, kv_heads=kv_heads, dim=dim)
        if vdim != dim:
            raise LoadError(f"config.json: {where} has values of size {vdim} and keys of size {dim}; its values are "
                            f"the keys")
        if heads % kv_heads:
            raise LoadError(f"config.json: {where} has {heads} query heads, no multiple of {kv_heads} key/value heads")
        if not scale > 0.0:
            raise LoadError(f"config.json: {where} mixer scale must be positive, got {scale}")
        mask = _section(r, "mask", where, required=False)
        chunk = mask.integer("size", None) if mask is not None else None
        if chunk is not None and chunk <= 0:
            raise LoadError(f"config.json: {where} mask size must be positive, got {chunk}")
        rot = _section(r, "rot", where, required=False)
        rotation = None
        if rot is not None:
            dims, base = rot.integer("dims", dim), rot.number("base")
            scaling = _section(rot, "scaling", where + " rot", required=False)
            factor = scaling.number("factor", 1.0) if scaling is not None else 1.0
            if dims <= 0 or dims % 2 or dims > dim:
                raise LoadError(f"config.json: {where} rotates {dims} dimensions of a head of {dim}: an even number "
                                f"up to the head's size is needed")
            if not base > 0.0 or not factor > 0.0:
                raise LoadError(f"config.json: {where} rot base and scaling factor must be positive")
            rotation = RotationConfig(dims, base, factor)
        return ChunkedAttentionMixerConfig(heads, kv_heads, dim, scale, chunk, rotation)

    @staticmethod
    def _mingru(r: ConfigReader, where: str) -> MinGruMixerConfig:
        width = r.integer("width")
        _positive(where, width=width)
        return MinGruMixerConfig(width)

    @staticmethod
    def _mlp(r: Optional[ConfigReader], where: str) -> Optional[DenseFfConfig]:
        if r is None:
            return None
        kind = r.string("kind")
        if kind != "dense":
            raise UnsupportedError(f"config.json: {where} has a feed-forward of kind '{kind}' (supported: dense)")
        ff = r.integer("ff")
        if ff <= 0:
            raise LoadError(f"config.json: {where} mlp ff must be positive, got {ff}")
        return DenseFfConfig(ff)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "TopapelConfig":
        r = ConfigReader(values)
        vocab, width = r.integer("vocab"), r.integer("width")
        if vocab <= 0 or width <= 0:
            raise LoadError(f"config.json: vocab and width must be positive, got {vocab} and {width}")
        eps = _section(r, "norm", "the model").number("eps")
        if not eps > 0.0:
            raise LoadError(f"config.json: norm eps must be positive, got {eps}")
        embedding = _section(r, "embedding", "the model", required=False)
        embedding_scale = embedding.number("scale", 1.0) if embedding is not None else 1.0
        logit_scale = r.number("logit_scale", 1.0)
        softcap = r.number("logit_softcap", None)
        if softcap is not None and not softcap > 0.0:
            raise LoadError(f"config.json: logit_softcap must be positive, got {softcap}")
        entries = r.raw("layers")
        if not isinstance(entries, list) or not entries:
            raise LoadError("config.json: 'layers' must be a non-empty list")
        readers = {"lightning": cls._lightning, "attention": cls._attention, "mingru": cls._mingru}
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
            layers.append(TopapelLayerConfig(kind, mixer, cls._mlp(_section(layer, "mlp", where, required=False), where)))
        max_positions = r.integer("max_positions", DEFAULT_MAX_POSITIONS)
        if max_positions <= 0:
            raise LoadError(f"config.json: max_positions must be positive, got {max_positions}")
        return cls(vocab, width, eps, embedding_scale, logit_scale, softcap, max_positions, tuple(layers))
