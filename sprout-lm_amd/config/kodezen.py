"""Configuration of the Kodezen decoder: a list of pre-norm layers, each with one of three mixers (two state-space mixers
and softmax attention whose heads' weights are mixed) behind a short convolution of the normed input, and a dense or routed
feed-forward."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, positive_float, positive_int

_WHAT = "Invalid Kodezen config: "


def _section(raw: Mapping, key: str, where: str, optional: bool = False):
    value = raw.get(key)
    if value is None and optional:
        return None
    if not isinstance(value, Mapping):
        raise ConfigError(f"{_WHAT}{where}{key} must be an object, got {value!r}.")
    return value


def _count(raw: Mapping, key: str, where: str, least: int = 1) -> int:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, int) or value < least:
        raise ConfigError(f"{_WHAT}{where}{key} must be an integer of at least {least}, got {value!r}.")
    return value


def _number(raw: Mapping, key: str, where: str) -> float:
    value = raw.get(key)
    if isinstance(value, bool) or not isinstance(value, (int, float)) or not math.isfinite(value) or value <= 0:
        raise ConfigError(f"{_WHAT}{where}{key} must be a positive finite number, got {value!r}.")
    return float(value)


@dataclass(frozen=True)
class DualitySizes:
    """Mixer "mamba2": heads of vdim values over `groups` shared B and C of `state` numbers; a convolution of `conv` taps;
    the gated output is normed in `norm_groups` parts."""

    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "DualitySizes":
        heads, vdim, groups = _count(raw, "heads", where), _count(raw, "vdim", where), _count(raw, "groups", where)
        parts = _count(raw, "norm_groups", where)
        if heads % groups:
            raise ConfigError(f"{_WHAT}{where}heads {heads} are no whole multiple of groups {groups}.")
        if (heads * vdim) % parts:
            raise ConfigError(f"{_WHAT}{where}{heads * vdim} values do not fall into {parts} equal parts.")
        return cls(heads, vdim, _count(raw, "state", where), groups, _count(raw, "conv", where), parts)

    def to_dict(self) -> dict:
        return {"conv": self.conv, "groups": self.groups, "heads": self.heads, "norm_groups": self.norm_groups,
                "state": self.state, "vdim": self.vdim}


@dataclass(frozen=True)
class ScanSizes:
    """Mixer "mamba1": `inner` channels with `state` states each, step sizes through a bottleneck of dt_rank numbers."""

    inner: int
    state: int
    dt_rank: int
    conv: int

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "ScanSizes":
        return cls(_count(raw, "inner", where), _count(raw, "state", where), _count(raw, "dt_rank", where),
                   _count(raw, "conv", where))

    def to_dict(self) -> dict:
        return {"conv": self.conv, "dt_rank": self.dt_rank, "inner": self.inner, "state": self.state}


@dataclass(frozen=True)
class AttentionSizes:
    """Mixer "attention".  window None: every earlier key is seen; else the last `window` and the first `keep_first`."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    conv: int
    rot_dims: int
    rot_base: float
    window: int | None
    keep_first: int

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "AttentionSizes":
        heads, kv_heads, dim, vdim = (_count(raw, k, where) for k in ("heads", "kv_heads", "dim", "vdim"))
        if heads % kv_heads:
            raise ConfigError(f"{_WHAT}{where}heads {heads} are no whole multiple of kv_heads {kv_heads}.")
        if vdim != dim:
            raise ConfigError(f"{_WHAT}{where}the values are the keys, so vdim {vdim} must equal dim {dim}.")
        rot = _section(raw, "rot", where)
        dims = _count(rot, "dims", where + "rot.", 0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"{_WHAT}{where}rot.dims must be even and at most dim {dim}, got {dims}.")
        mask = _section(raw, "mask", where, optional=True)
        window = None if mask is None else _count(mask, "size", where + "mask.")
        keep = 0 if mask is None else _count(mask, "keep_first", where + "mask.", 0)
        return cls(heads, kv_heads, dim, vdim, _number(raw, "scale", where), _count(raw, "conv", where), dims,
                   _number(rot, "base", where + "rot."), window, keep)

    def to_dict(self) -> dict:
        out = {"conv": self.conv, "dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads,
               "rot": {"base": self.rot_base, "dims": self.rot_dims}, "scale": self.scale, "vdim": self.vdim}
        if self.window is not None:
            out["mask"] = {"keep_first": self.keep_first, "size": self.window}
        return out


_MIXERS = {"mamba2": DualitySizes, "mamba1": ScanSizes, "attention": AttentionSizes}


@dataclass(frozen=True)
class FeedForwardSizes:
    """kind "dense": `ff` inner numbers.  kind "moe": `experts` experts of `ff` inner numbers, `top` of them a token."""

    kind: str
    ff: int
    experts: int = 0
    top: int = 0

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "FeedForwardSizes":
        kind = raw.get("kind")
        if kind == "dense":
            return cls("dense", _count(raw, "ff", where))
        if kind == "moe":
            router = _section(raw, "router", where)
            experts, top = _count(router, "experts", where + "router."), _count(router, "top", where + "router.")
            if top > experts:
                raise ConfigError(f"{_WHAT}{where}router.top {top} exceeds the {experts} experts.")
            return cls("moe", _count(_section(raw, "expert", where), "ff", where + "expert."), experts, top)
        raise ConfigError(f"{_WHAT}{where}kind must be 'dense' or 'moe', got {kind!r}.")

    def to_dict(self) -> dict:
        if self.kind == "dense":
            return {"ff": self.ff, "kind": "dense"}
        return {"expert": {"ff": self.ff}, "kind": "moe", "router": {"experts": self.experts, "top": self.top}}


@dataclass(frozen=True)
class KodezenLayer:
    kind: str                        # "mamba2", "mamba1" or "attention"
    mixer: object
    ff: FeedForwardSizes | None      # None for a layer without feed-forward

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else self.ff.to_dict(), "type": self.kind}


@dataclass(frozen=True)
class KodezenConfig(ModelConfig):
    """Every size and constant of a Kodezen model, as config.json gives them; nothing has a default."""

    architecture: ClassVar[str] = "Kodezen"

    vocab: int
    width: int
    eps: float
    embedding_scale: float
    canon_taps: int
    layers: tuple[KodezenLayer, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "KodezenConfig":
        if not isinstance(raw, Mapping):
            raise ConfigError(_WHAT + "expected a JSON object.")
        if raw.get("architecture") != cls.architecture:
            raise ConfigError(f"Not a Kodezen config: architecture is {raw.get('architecture')!r}.")
        vocab, width = positive_int(raw, "vocab"), positive_int(raw, "width")
        eps = positive_float(_section(raw, "norm", ""), "eps")
        scale = _number(_section(raw, "embedding", ""), "scale", "embedding.")
        taps = _count(_section(raw, "canon", ""), "taps", "canon.")
        entries = raw.get("layers")
        if not isinstance(entries, list) or not entries:
            raise ConfigError(_WHAT + "layers must be a non-empty list.")
        layers = []
        for i, entry in enumerate(entries):
            where = f"layers[{i}]."
            if not isinstance(entry, Mapping):
                raise ConfigError(f"{_WHAT}layers[{i}] must be an object.")
            kind = entry.get("type")
            if kind not in _MIXERS:
                raise ConfigError(f"{_WHAT}{where}type {kind!r} is no mixer of this design {tuple(_MIXERS)}.")
            mixer = _MIXERS[kind].parse(_section(entry, "mixer", where), where + "mixer.")
            mlp = _section(entry, "mlp", where, optional=True)
            layers.append(KodezenLayer(kind, mixer, None if mlp is None else FeedForwardSizes.parse(mlp, where + "mlp.")))
        return cls(vocab, width, eps, scale, taps, tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "canon": {"taps": self.canon_taps}, "embedding": {"scale": self.embedding_scale},
                "layers": [layer.to_dict() for layer in self.layers], "norm": {"eps": self.eps}, "vocab": self.vocab,
                "width": self.width}
