"""Rotary position encoding, half-split ("neox") pairing (reference: rope, src/qwen.ts:81-92)."""
from __future__ import annotations

import torch

from .base import PositionEncoding, register_part


@register_part("position", "rotary_neox")
class NeoxRotary(PositionEncoding):
    """Pair (d, d + rotary_dim/2) of a head turns by position * theta^(-2d / rotary_dim).

    `scaling` (None, or factor / original / fast / slow): frequencies are blended between f_d and f_d / factor along a
    ramp over the pair index d, and cosine and sine are multiplied by `magnitude` = 0.1 ln(factor) + 1 ("YaRN"): with
    turns(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(turns(fast)), 0), hi =
    min(ceil(turns(slow)), rotary_dim - 1) and ramp_d = clamp((d - lo) / max(hi - lo, 0.001), 0, 1) pair d turns by
    position * (f_d / factor * ramp_d + f_d * (1 - ramp_d)).

    The table of inverse frequencies is computed in float64 and kept in float32; angles, sines
    and cosines are float32 in the kernel.  For float32 models the part also keeps what the float32
    table lost (`inv_freq_tail`), and the kernel computes angle, sine and cosine in float64: a float32
    angle is off by up to position * 6e-8, more than every other rounding of that path together once
    positions reach the thousands.
    """

    graph_safe = True

    graph_safe_portions = True
    pairing = "halves"      # which dimensions turn together, as the kernels name it (ops.ROTARY_PAIRINGS)

    def __init__(self, head_dim: int, theta: float, rotary_dim: int | None = None, scaling: dict | None = None):
        import math
        self.head_dim, self.theta = head_dim, theta
        self.rotary_dim = head_dim if rotary_dim is None else rotary_dim
        if self.rotary_dim % 2 or not 0 < self.rotary_dim <= head_dim:
            raise ValueError(f"rotary_dim {self.rotary_dim} must be even and at most head_dim {head_dim}.")
        self.scaling = dict(scaling) if scaling else None
        self.magnitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0 if self.scaling else 1.0
        self.inv_freq = None
        self.inv_freq_tail = None

    def frequencies(self) -> torch.Tensor:
        """The exact (float64) frequency of every pair."""
        import math
        n = self.rotary_dim
        d = torch.arange(n // 2, dtype=torch.float64)
        freq = float(self.theta) ** (-2.0 * d / n)
        if not self.scaling:
            return freq
        factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
        turns = lambda t: n * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(float(self.theta)))
        lo = max(math.floor(turns(float(self.scaling["fast"]))), 0)
        hi = min(math.ceil(turns(float(self.scaling["slow"]))), n - 1)
        ramp = ((d - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return freq / factor * ramp + freq * (1.0 - ramp)

    def prepare(self, device, dtype):
        exact = self.frequencies()
        self.inv_freq = exact.to(torch.float32).to(device)
        if dtype == torch.float32:
            self.inv_freq_tail = (exact - exact.to(torch.float32).to(torch.float64)).to(torch.float32).to(device)

    def table(self, ctx) -> torch.Tensor:
        """(cosine, sine) of every token's angles, float32 [T, rotary_dim / 2, 2]: the same in every layer, so
        the first layer of a step that asks computes it and the others find it in the step's context."""
        from .. import ops
        scaling = tuple(sorted(self.scaling.items())) if self.scaling else ()
        key = ("rotary_neox", self.rotary_dim, float(self.theta), scaling)
        found = ctx.shared.get(key)
        if found is None:
            name = f"rotation_table_{self.rotary_dim}_{float(self.theta)!r}" + (f"_{hash(scaling) & 0xffffffff:x}" if scaling else "")
            found = ctx.buffer(name, (ctx.n_tokens, self.rotary_dim // 2, 2), torch.float32)
            ops.rope_table(ctx.positions, self.inv_freq, found, inv_freq_tail=self.inv_freq_tail, magnitude=self.magnitude)
            ctx.shared[key] = found
        return found


@register_part("position", "rotary_interleaved")
class InterleavedRotary(PositionEncoding):
    """Neighbours (2i, 2i + 1) of the first `rotary_dim` numbers turn by position * f_i, f_i = theta^(-2i / rotary_dim).

    `scaling` (None, or factor / original / fast / slow): frequencies are blended between f_i and f_i / factor
    along a ramp over the pair index, and cosine and sine are multiplied by `magnitude` = 0.1 ln(factor) + 1
    ("YaRN").  With turns(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), lo = max(floor(turns(fast)), 0),
    hi = min(ceil(turns(slow)), rotary_dim - 1) and ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the
    frequency of pair i is f_i / factor * ramp_i + f_i * (1 - ramp_i).

    The table `freq` is float64 on the device; the kernels that turn (the latent mixer's) compute the angle in
    float32 for bfloat16 models and in float64 for float32 models."""

    graph_safe = True

    graph_safe_portions = True
    pairing = "interleaved"

    def __init__(self, rotary_dim: int, theta: float, scaling: dict | None = None):
        import math
        if rotary_dim % 2 or rotary_dim < 0:
            raise ValueError(f"rotary_dim {rotary_dim} must be even.")
        self.rotary_dim, self.theta, self.scaling = rotary_dim, float(theta), dict(scaling) if scaling else None
        self.magnitude = 0.1 * math.log(float(self.scaling["factor"])) + 1.0 if self.scaling else 1.0
        self.freq = None
        self.inv_freq = None

    def frequencies(self) -> torch.Tensor:
        import math
        n = self.rotary_dim
        i = torch.arange(n // 2, dtype=torch.float64)
        freq = self.theta ** (-2.0 * i / max(n, 1))
        if not self.scaling:
            return freq
        factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
        turns = lambda t: n * math.log(original / (2.0 * math.pi * t)) / (2.0 * math.log(self.theta))
        lo = max(math.floor(turns(float(self.scaling["fast"]))), 0)
        hi = min(math.ceil(turns(float(self.scaling["slow"]))), n - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
        return freq / factor * ramp + freq * (1.0 - ramp)

    def prepare(self, device, dtype):
        exact = self.frequencies() if self.rotary_dim else torch.zeros(1, dtype=torch.float64)
        self.freq = exact.to(device)
        self.inv_freq = exact.to(torch.float32).to(device)


@register_part("position", "none")
class NoPosition(PositionEncoding):
    """No position encoding: queries and keys are used as projected."""

    rotary_dim = 0
    pairing = "halves"      # nothing turns; the kernels are asked for the pairing they have

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, head_dim: int = 0):
        self.head_dim = head_dim
        self.inv_freq = None

    def prepare(self, device, dtype):
        self.inv_freq = torch.zeros(1, dtype=torch.float32, device=device)
