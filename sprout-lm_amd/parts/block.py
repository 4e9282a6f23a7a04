"""Arrangement of parts in a layer (reference: src/qwen.ts:164-202)."""
from __future__ import annotations

from .base import Block, register_part


@register_part("block", "pre_norm")
class PreNormBlock(Block):
    """x += mixer(norm(x)); x += feed_forward(norm(x)).  The residual stream x is float32.  `ffn` (and its norm) may
    be absent: the layer is then its mixer alone.  `mixer_conv`: a part that stands between the norm and the mixer (a
    short convolution over time, which keeps its last inputs per request): the mixer reads mixer_conv(norm(x))."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None, mixer_conv=None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn, self.mixer_conv = mixer_norm, mixer, ffn_norm, ffn, mixer_conv

    def parts(self):
        named = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.mixer_conv is not None:
            named["mixer_conv"] = self.mixer_conv
        if self.ffn is not None:
            named.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})
        return named

    def forward(self, ctx, residual, caches):
        T, H = residual.shape
        cache = caches.get("mixer")
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        if self.mixer_conv is not None:
            self.mixer_norm.forward(ctx, residual, h)
            mixed_in = ctx.buffer("normed_conv", (T, H), ctx.act_dtype)
            self.mixer_conv.forward(ctx, h, mixed_in, caches.get("mixer_conv"))
            self.mixer.forward(ctx, mixed_in, residual, cache)
        elif not self.mixer.forward_from_residual(ctx, self.mixer_norm, residual, cache):
            self.mixer_norm.forward(ctx, residual, h)
            self.mixer.forward(ctx, h, residual, cache)
        if self.ffn is None:
            return
        if not self.ffn.forward_from_residual(ctx, self.ffn_norm, residual):
            self.ffn_norm.forward(ctx, residual, h)
            self.ffn.forward(ctx, h, residual)


@register_part("block", "parallel")
class ParallelBlock(Block):
    """x += mixer(norm_a(x)) + feed_forward(norm_b(x)): both norms read the same x, so both are taken before
    either part adds into the float32 residual stream.  `ffn` (and its norm) may be absent."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None):
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        named = {"mixer_norm": self.mixer_norm, "mixer": self.mixer}
        if self.ffn is not None:
            named.update({"ffn_norm": self.ffn_norm, "ffn": self.ffn})
        return named

    def forward(self, ctx, residual, caches):
        T, H = residual.shape
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        if self.ffn is None:
            self.mixer_norm.forward(ctx, residual, h)
        else:
            h2 = ctx.buffer("normed_ffn", (T, H), ctx.act_dtype)
            pair = getattr(self.mixer_norm, "forward_pair", None)      # norms that share their statistics take one pass
            if pair is None or not pair(ctx, self.ffn_norm, residual, h, h2):
                self.mixer_norm.forward(ctx, residual, h)
                self.ffn_norm.forward(ctx, residual, h2)
        self.mixer.forward(ctx, h, residual, caches.get("mixer"))
        if self.ffn is not None:
            self.ffn.forward(ctx, h2, residual)


@register_part("block", "parallel_scaled")
class ScaledParallelBlock(Block):
    """x += scale_a(mixer(norm(x))) + scale_b(feed_forward(norm(x))): ONE norm whose output both sublayers read, and each
    sublayer's result goes through a part of its own (a learned vector, a constant) before the sum.  The sublayers add
    into float32 rows of their own, which are cleared first; `ffn` (and its scale) may be absent."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, mixer_norm, mixer, mixer_scale, ffn=None, ffn_scale=None):
        self.mixer_norm, self.mixer, self.mixer_scale, self.ffn, self.ffn_scale = mixer_norm, mixer, mixer_scale, ffn, ffn_scale

    def parts(self):
        named = {"mixer_norm": self.mixer_norm, "mixer": self.mixer, "mixer_scale": self.mixer_scale}
        if self.ffn is not None:
            named.update({"ffn": self.ffn, "ffn_scale": self.ffn_scale})
        return named

    def forward(self, ctx, residual, caches):
        import torch
        T, H = residual.shape
        h = ctx.buffer("normed", (T, H), ctx.act_dtype)
        self.mixer_norm.forward(ctx, residual, h)
        both = ctx.buffer("branches", (2, T, H), torch.float32)
        if self.ffn is None:
            both[0].zero_()
            self.mixer.forward(ctx, h, both[0], caches.get("mixer"))
            self.mixer_scale.add(ctx, residual, both[0])
            return
        both.zero_()
        self.mixer.forward(ctx, h, both[0], caches.get("mixer"))
        self.ffn.forward(ctx, h, both[1])
        self.mixer_scale.add(ctx, residual, both[0], self.ffn_scale, both[1])
