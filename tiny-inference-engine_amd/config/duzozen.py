"""Typed configuration of the Duzozen decoder, read from its config.json.

Duzozen describes itself layer by layer: ``layers`` is a list whose entries name a mixer type, the mixer's sizes
and constants, and a feed-forward (or none). Nothing about a layer is assumed from another layer: head counts,
head sizes, windows, score scale and cap, and the kind of feed-forward may all differ. Keys read:

    architecture          "Duzozen"
    vocab, width          sizes of the embedding table / the residual stream
    norm.eps              the eps of every RMS norm
    max_positions         optional: the longest sequence (default 131072; the design itself has no limit)
    layers[i].type        "attention"
    layers[i].mixer       heads, kv_heads, dim, vdim, scale, softcap (optional), mask.size (optional), v_mix (optional)
    layers[i].mlp         null, or kind "dense" with ff, or kind "moe" with expert.ff and router.{experts, identity,
                          top, groups.{count, keep}}
"""

from __future__ import annotations

import dataclasses
import math
from typing import Any, Mapping, Optional, Tuple

from ..errors import LoadError, UnsupportedError
from .base import ConfigReader

DEFAULT_MAX_POSITIONS = 131072


def _section(reader: ConfigReader, key: str, where: str, required: bool = True) -> Optional[ConfigReader]:
    value = reader.raw(key)
    if value is None:
        if required:
            raise LoadError(f"config.json: {where} has no '{key}'")
        return None
    if not isinstance(value, Mapping):
        raise LoadError(f"config.json: {where} '{key}' must be an object, got {value!r}")
    return ConfigReader(value, f"config.json {where} {key}")


@dataclasses.dataclass(frozen=True)
class AttentionMixerConfig:
    heads: int
    kv_heads: int
    dim: int                      # size of a query / key head
    vdim: int                     # size of a value head
    scale: float                  # the scores' factor
    softcap: Optional[float]      # scores become cap * tanh(score / cap); None: uncapped
    window: Optional[int]         # a query sees itself and the window - 1 positions before it; None: all
    v_mix: bool                   # values blended with those of the first layer that says so


@dataclasses.dataclass(frozen=True)
class DenseMlpConfig:
    ff: int


@dataclasses.dataclass(frozen=True)
class RoutedMlpConfig:
    expert_ff: int
    experts: int                  # experts with weights
    identity: int                 # further router outputs whose expert returns its input
    top: int
    group_count: int
    group_keep: int


@dataclasses.dataclass(frozen=True)
class DuzozenLayerConfig:
    mixer: AttentionMixerConfig
    mlp: Any                      # None, DenseMlpConfig or RoutedMlpConfig


@dataclasses.dataclass(frozen=True)
class DuzozenConfig:
    vocab: int
    width: int
    norm_eps: float
    max_positions: int
    layers: Tuple[DuzozenLayerConfig, ...]

    @staticmethod
    def _mixer(r: ConfigReader, where: str) -> AttentionMixerConfig:
        heads = r.integer("heads")
        kv_heads = r.integer("kv_heads", heads)
        dim = r.integer("dim")
        vdim = r.integer("vdim", dim)
        scale = r.number("scale")
        softcap = r.number("softcap", None)
        mask = _section(r, "mask", where, required=False)
        window = mask.integer("size", None) if mask is not None else None
        for name, value in (("heads", heads), ("kv_heads", kv_heads), ("dim", dim), ("vdim", vdim)):
            if value <= 0:
                raise LoadError(f"config.json: {where} mixer {name} must be positive, got {value}")
        if heads % kv_heads:
            raise LoadError(f"config.json: {where} has {heads} query heads, no multiple of {kv_heads} key/value heads")
        if not scale > 0.0:
            raise LoadError(f"config.json: {where} mixer scale must be positive, got {scale}")
        if softcap is not None and not softcap > 0.0:
            raise LoadError(f"config.json: {where} mixer softcap must be positive, got {softcap}")
        if window is not None and window <= 0:
            raise LoadError(f"config.json: {where} mask size must be positive, got {window}")
        return AttentionMixerConfig(heads, kv_heads, dim, vdim, scale, softcap, window, r.boolean("v_mix", False))

    @staticmethod
    def _mlp(r: Optional[ConfigReader], where: str):
        if r is None:
            return None
        kind = r.string("kind")
        if kind == "dense":
            ff = r.integer("ff")
            if ff <= 0:
                raise LoadError(f"config.json: {where} mlp ff must be positive, got {ff}")
            return DenseMlpConfig(ff)
        if kind != "moe":
            raise UnsupportedError(f"config.json: {where} has a feed-forward of kind '{kind}' (supported: dense, moe)")
        expert = _section(r, "expert", where + " mlp")
        router = _section(r, "router", where + " mlp")
        groups = _section(router, "groups", where + " mlp router", required=False)
        experts, identity = router.integer("experts"), router.integer("identity", 0)
        top = router.integer("top")
        count = groups.integer("count", 1) if groups is not None else 1
        keep = groups.integer("keep", count) if groups is not None else 1
        ff = expert.integer("ff")
        if experts <= 0 or identity < 0 or ff <= 0:
            raise LoadError(f"config.json: {where} needs positive experts and expert ff and no negative identity count")
        total = experts + identity
        if count <= 0 or total % count or not 0 < keep <= count:
            raise LoadError(f"config.json: {where} cannot form {count} equal groups of {total} router outputs and keep {keep}")
        if not 0 < top <= keep * (total // count):
            raise LoadError(f"config.json: {where} chooses {top} experts out of {keep} groups of {total // count}")
        return RoutedMlpConfig(ff, experts, identity, top, count, keep)

    @classmethod
    def from_json(cls, values: Mapping[str, Any]) -> "DuzozenConfig":
        r = ConfigReader(values)
        vocab, width = r.integer("vocab"), r.integer("width")
        if vocab <= 0 or width <= 0:
            raise LoadError(f"config.json: vocab and width must be positive, got {vocab} and {width}")
        eps = _section(r, "norm", "the model").number("eps")
        if not eps > 0.0 or not math.isfinite(eps):
            raise LoadError(f"config.json: norm eps must be positive, got {eps}")
        entries = r.raw("layers")
        if not isinstance(entries, list) or not entries:
            raise LoadError("config.json: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layer {i}"
            if not isinstance(entry, Mapping):
                raise LoadError(f"config.json: {where} must be an object")
            layer = ConfigReader(entry, f"config.json {where}")
            kind = layer.string("type")
            if kind != "attention":
                raise UnsupportedError(f"config.json: {where} has a mixer of type '{kind}' (supported: attention)")
            mixer = cls._mixer(_section(layer, "mixer", where), where)
            layers.append(DuzozenLayerConfig(mixer, cls._mlp(_section(layer, "mlp", where, required=False), where)))
        mixing = [l.mixer for l in layers if l.mixer.v_mix]
        if any((m.kv_heads, m.vdim) != (mixing[0].kv_heads, mixing[0].vdim) for m in mixing):
            raise LoadError("config.json: layers that blend their values (v_mix) must agree in kv_heads and vdim")
        max_positions = r.integer("max_positions", DEFAULT_MAX_POSITIONS)
        if max_positions <= 0:
            raise LoadError(f"config.json: max_positions must be positive, got {max_positions}")
        return cls(vocab, width, eps, max_positions, tuple(layers))
