"""Configuration of the Morarax decoder: a list of layers, each with one of three mixers (softmax attention, a gated
linear recurrence, retention) beside an optional dense feed-forward, under one norm."""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Any, ClassVar, Mapping

from .base import ConfigError, ModelConfig, positive_float, positive_int

_WHAT = "Invalid Morarax config: "


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
class Rotation:
    """`dims` numbers of a head turn (0: none) with frequencies base^(-2i/dims); `scaling`: (factor, original, fast,
    slow) of the blended frequencies, or None."""

    dims: int
    base: float
    scaling: tuple | None = None

    @classmethod
    def parse(cls, raw: Mapping, where: str, dim: int) -> "Rotation":
        dims = _count(raw, "dims", where, 0)
        if dims % 2 or dims > dim:
            raise ConfigError(f"{_WHAT}{where}dims must be even and at most dim {dim}, got {dims}.")
        scaling = _section(raw, "scaling", where, optional=True)
        if scaling is not None:
            scaling = tuple(_number(scaling, k, where + "scaling.") for k in ("factor", "original", "fast", "slow"))
        return cls(dims, _number(raw, "base", where), scaling)

    def scaling_dict(self):
        return None if self.scaling is None else dict(zip(("factor", "original", "fast", "slow"), self.scaling))

    def to_dict(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.scaling is not None:
            out["scaling"] = self.scaling_dict()
        return out


@dataclass(frozen=True)
class AttentionSizes:
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot: Rotation

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "AttentionSizes":
        heads, kv_heads, dim = _count(raw, "heads", where), _count(raw, "kv_heads", where), _count(raw, "dim", where)
        if heads % kv_heads:
            raise ConfigError(f"{_WHAT}{where}heads {heads} are no whole multiple of kv_heads {kv_heads}.")
        return cls(heads, kv_heads, dim, _count(raw, "vdim", where), _number(raw, "scale", where),
                   Rotation.parse(_section(raw, "rot", where), where + "rot.", dim))

    def to_dict(self) -> dict:
        return {"dim": self.dim, "heads": self.heads, "kv_heads": self.kv_heads, "rot": self.rot.to_dict(),
                "scale": self.scale, "vdim": self.vdim}


@dataclass(frozen=True)
class RecurrenceSizes:
    width: int
    blocks: int
    conv: int

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "RecurrenceSizes":
        width, blocks = _count(raw, "width", where), _count(raw, "blocks", where)
        if width % blocks:
            raise ConfigError(f"{_WHAT}{where}width {width} does not fall into {blocks} equal parts.")
        return cls(width, blocks, _count(raw, "conv", where))

    def to_dict(self) -> dict:
        return {"blocks": self.blocks, "conv": self.conv, "width": self.width}


@dataclass(frozen=True)
class RetentionSizes:
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot: Rotation

    @classmethod
    def parse(cls, raw: Mapping, where: str) -> "RetentionSizes":
        heads, dim = _count(raw, "heads", where), _count(raw, "dim", where)
        decay = raw.get("decay")
        if (not isinstance(decay, list) or len(decay) != heads or
                any(isinstance(d, bool) or not isinstance(d, (int, float)) or not 0.0 <= d <= 1.0 for d in decay)):
            raise ConfigError(f"{_WHAT}{where}decay must list one number in [0, 1] per head, got {decay!r}.")
        return cls(heads, dim, _count(raw, "vdim", where), tuple(float(d) for d in decay),
                   Rotation.parse(_section(raw, "rot", where), where + "rot.", dim))

    def to_dict(self) -> dict:
        return {"decay": list(self.decay), "dim": self.dim, "heads": self.heads, "rot": self.rot.to_dict(), "vdim": self.vdim}


_MIXERS = {"attention": AttentionSizes, "rglru": RecurrenceSizes, "retention": RetentionSizes}


@dataclass(frozen=True)
class MoraraxLayer:
    kind: str                 # "attention", "rglru" or "retention"
    mixer: object
    ff: int | None            # the dense feed-forward's inner size, None for a layer without one

    def to_dict(self) -> dict:
        return {"mixer": self.mixer.to_dict(), "mlp": None if self.ff is None else {"ff": self.ff, "kind": "dense"},
                "type": self.kind}


@dataclass(frozen=True)
class MoraraxConfig(ModelConfig):
    """Every size and constant of a Morarax model, as config.json gives them; nothing has a default."""

    architecture: ClassVar[str] = "Morarax"

    vocab: int
    width: int
    eps: float
    residual_mult: float
    logit_scale: float
    layers: tuple[MoraraxLayer, ...]

    @property
    def vocab_size(self) -> int:
        return self.vocab

    @property
    def hidden_size(self) -> int:
        return self.width

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "MoraraxConfig":
        if not isinstance(raw, Mapping):
            raise ConfigError(_WHAT + "expected a JSON object.")
        if raw.get("architecture") != cls.architecture:
            raise ConfigError(f"Not a Morarax config: architecture is {raw.get('architecture')!r}.")
        vocab, width = positive_int(raw, "vocab"), positive_int(raw, "width")
        eps = positive_float(_section(raw, "norm", ""), "eps")
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
            if mlp is not None and mlp.get("kind") != "dense":
                raise ConfigError(f"{_WHAT}{where}mlp.kind must be 'dense', got {mlp.get('kind')!r}.")
            layers.append(MoraraxLayer(kind, mixer, None if mlp is None else _count(mlp, "ff", where + "mlp.")))
        return cls(vocab, width, eps, _number(raw, "residual_mult", ""), _number(raw, "logit_scale", ""), tuple(layers))

    def to_dict(self) -> dict:
        return {"architecture": self.architecture, "layers": [layer.to_dict() for layer in self.layers],
                "logit_scale": self.logit_scale, "norm": {"eps": self.eps}, "residual_mult": self.residual_mult,
                "vocab": self.vocab, "width": self.width}
