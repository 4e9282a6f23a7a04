"""Grouped-query attention whose heads' softmax weights are mixed by a learned matrix after the softmax, with a short
convolution on q and k, the keys themselves as values, and a window that keeps a sequence's first keys."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import PagedKVSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part
from .conv import ShortConv
from .sink_attention import padded_width


@register_part("mixer", "mixed_heads_attention")
class MixedHeadsAttention(Mixer):
    """q = conv(W_q h), k = conv(W_k h): a causal convolution of `taps` taps per channel, no bias (one tap: a factor per channel).  The
    values are the keys as they leave the convolution.  Every q and k head is then RMS-normed over `dim` with a weight of
    that size shared by the heads (`eps` inside the root), and `position` (neighbouring pairs) turns its first numbers.
    score = (q . k) * scale; position i sees j <= i with i - j < window (None: all) or j < keep_first; ordinary softmax.
    With P_g the weights of head g, head n's output is sum_g talk[n, g] P_g V_(kv(n)), and W_o mixes the heads' outputs.

    The softmax weights never leave the attention kernels, and the mix is linear in them: every (query head g, value head c)
    pair runs as a head of its own (heads * kv_heads of them over kv_heads^2 key/value heads: the keys of a, the values of
    c), and head n's output is sum_g talk[n, g] O[g, kv(n)].  The cache holds a key kv_heads times for that.

    `tensors`: local names of W_q, W_k, the suffixes of their convolutions and norms, the mixing matrix and W_o.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, scale: float, position, taps: int, eps: float,
                 window: int | None = None, keep_first: int = 0, page_tokens: int | None = None,
                 tensors: tuple = ("q", "k", ".conv", ".norm", "talk", "o")):
        if min(hidden, heads, kv_heads, dim, taps) <= 0 or heads % kv_heads:
            raise ConfigError(f"Attention needs positive sizes and heads in whole groups, got heads={heads} kv_heads={kv_heads} dim={dim}.")
        if window is not None and window <= 0 or keep_first < 0:
            raise ConfigError(f"A window is positive and the kept first keys are not negative, got {window!r} and {keep_first!r}.")
        rotary = getattr(position, "rotary_dim", 0)
        if rotary and (getattr(position, "pairing", None) != "interleaved" or rotary > dim or rotary % 2):
            raise ConfigError(f"This mixer turns the first {rotary} numbers of a head of {dim} in neighbouring pairs; the position "
                              f"encoding must pair them so and fit.")
        self.width = padded_width(dim, dim)
        try:
            ops.check_attention_sizes(heads * kv_heads, kv_heads * kv_heads, self.width)
        except ops.KernelError as error:
            raise ConfigError(str(error)) from None
        self.hidden, self.heads, self.kv_heads, self.dim, self.scale = hidden, heads, kv_heads, dim, float(scale)
        self.position, self.taps, self.eps, self.window = position, taps, float(eps), window
        self.keep_first = int(keep_first) if window is not None else 0
        self.page_tokens = page_tokens
        self.names = tuple(tensors)
        self.channels = (heads + kv_heads) * dim
        self.conv = ShortConv(self.channels, taps, tensor="conv")

    def cache_spec(self):
        spec = {"pages": PagedKVSpec(self.kv_heads * self.kv_heads, self.width, self.window, self.page_tokens,
                                     keep_first=self.keep_first)}
        if self.taps > 1:
            spec["inputs"] = self.conv.cache_spec()
        return spec

    def cache_elements_per_token(self) -> int:
        return 2 * self.kv_heads * self.kv_heads * self.width

    def flops(self, tokens: int, pairs: int = 0) -> float:
        projections = 2.0 * tokens * self.hidden * (2 * self.heads + self.kv_heads) * self.dim
        return projections + 4.0 * self.heads * self.kv_heads * self.dim * pairs

    def tensors(self):
        q, k, conv, norm, talk, o = self.names
        H, G, D = self.heads, self.kv_heads, self.dim
        out = {q: TensorSpec((H * D, self.hidden)), k: TensorSpec((G * D, self.hidden)),
               q + norm: TensorSpec((D,), "vector", "one_plus_normal"), k + norm: TensorSpec((D,), "vector", "one_plus_normal"),
               talk: TensorSpec((H, H), "vector", "one_plus_normal"), o: TensorSpec((self.hidden, H * D)),
               q + conv: TensorSpec((H * D, self.taps), "vector"), k + conv: TensorSpec((G * D, self.taps), "vector")}
        return out

    def bind(self, tensors):
        q, k, conv, norm, talk, o = self.names
        self.w_qk = torch.cat([tensors[q], tensors[k]], dim=0).contiguous()
        self.conv.bind({"conv": torch.cat([tensors[q + conv], tensors[k + conv]], dim=0).contiguous()})
        self.w_q_norm, self.w_k_norm = tensors[q + norm].contiguous(), tensors[k + norm].contiguous()
        self.talk = tensors[talk].to(torch.float32).contiguous()
        self.w_o = tensors[o]
        self.w = {}

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def subparts(self):
        return [self.position]

    def forward(self, ctx, h, residual, cache):
        T, H, G, D, W = h.shape[0], self.heads, self.kv_heads, self.dim, self.width
        pages = cache["pages"]
        raw = ctx.buffer("qk", (T, self.channels), ctx.act_dtype)
        ops.gemm(h, self.w_qk, raw)
        qk = ctx.buffer("qk_conv", (T, self.channels), ctx.act_dtype)
        self.conv.forward(ctx, raw, qk, cache.get("inputs"))
        queries = ctx.buffer("cross_q", (T, H * G * W), ctx.act_dtype)
        rotary = getattr(self.position, "rotary_dim", 0)
        writes = pages.writes
        ops.qk_cross_prepare(qk, H, G, D, W, self.w_q_norm, self.w_k_norm, self.eps, ctx.positions,
                             self.position.freq if rotary else None, rotary, queries,
                             slot_mapping=pages.slot_mapping if writes else None, k_pool=pages.k if writes else None,
                             v_pool=pages.v if writes else None)
        outputs = ctx.buffer("cross_o", (T, H * G * W), ctx.act_dtype)
        ops.attention(queries, H * G * W, pages.k, pages.v, pages.block_tables, ctx.attention, outputs, H * G, G * G, W,
                      self.window, self.scale, workspace=lambda n: ctx.buffer("attention_partials", (n,), torch.float32),
                      kind=ctx.attention_kind, keep_first=self.keep_first)
        mixed = ctx.buffer("attn", (T, H * D), ctx.act_dtype)
        ops.head_mix(outputs, self.talk, H, G, D, W, mixed)
        ops.gemm(mixed, self.w_o, residual, accumulate=True)
