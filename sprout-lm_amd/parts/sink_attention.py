"""Grouped-query attention with the extras some designs put around the softmax: heads whose keys and values differ
in width, a learned logit per head in the denominator, capped scores, blocks of positions that do not see each other,
norms over whole query and key rows, and values blended with an earlier layer's."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import PagedKVSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part

# the head sizes the matrix-core attention kernels take; a head is kept this wide in the cache, zeros behind
_KERNEL_WIDTHS = (16, 32, 48, 64, 80, 96, 128)


def padded_width(dim: int, vdim: int) -> int:
    """The width at which keys and values of `dim` and `vdim` numbers are both kept: the next head size the
    matrix-core kernels take, else the next multiple of 16 (float32 matrix cores up to 256), else as it is."""
    need = max(dim, vdim)
    for width in _KERNEL_WIDTHS:
        if need <= width:
            return width
    return -(-need // 16) * 16 if need <= 256 else need


@register_part("mixer", "sink_attention")
class SinkAttention(Mixer):
    """q = W_q h (+ b), k = W_k h (+ b), v = W_v h (+ b); head h of `heads` reads key/value head h // (heads / kv_heads).

    qk_norm: q and k are RMS-normed as whole rows (all heads at once) with weights of that length, `eps` inside the root.
    position: a PositionEncoding with "halves" pairing whose first `rotary_dim` numbers of every q and k head turn, or one
    that turns nothing.  score = (q . k) * scale; softcap c: score <- c * tanh(score / c).  mask_chunk n: position i sees
    j <= i with i // n == j // n only, blocks counted from position 0 of the sequence; window n: j > i - n.  sinks: the
    softmax's denominator also holds exp(sink_h), a tensor of one number per head that has no key and no value.
    value_mix: None, "first" (this layer's values are kept for the step under `value_key`) or "blend" (v <- (1 - l) v +
    l first, l the one-number tensor `blend`); the blended values are what is cached.  W_o mixes the heads' outputs.
    head_norm: after turning, every q and k head is divided by its root mean square over dim (`eps` inside the root, no
    weight).  sink_value: a constant logit in the denominator in place of learned ones (0.0: the denominator holds one
    more 1).  head_gate: head h's output is multiplied by sigmoid((W_g h)_h), W_g a tensor [heads, hidden] whose rows ride
    behind those of q, k and v in the one product (the last name of `tensors`).  A position encoding may scale its
    cosines and sines (`magnitude`).

    Keys (dim numbers) and values (vdim numbers) lie in the cache at one common width (`padded_width`), zeros behind, so
    the attention kernels see equal head sizes; W_o gets columns of zeros to match.  What a step does: one product for
    q, k, v (biases inside), `ops.qkv_prepare` (norms, rotation, blend, cache write), attention, the output product.

    `tensors`: local names of q, k, v, o, the biases' suffix, the q and k norm suffix, the blend factor and the sinks.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, kv_heads: int, dim: int, vdim: int, scale: float, position, qkv_bias: bool = False,
                 qk_norm: bool = False, eps: float = 0.0, softcap: float | None = None, mask_chunk: int | None = None,
                 window: int | None = None, sinks: bool = True, value_mix: str | None = None, value_key: str = "first_values",
                 page_tokens: int | None = None, head_norm: bool = False, sink_value: float | None = None,
                 head_gate: bool = False,
                 tensors: tuple = ("q", "k", "v", "o", ".b", ".norm", "vmix", "sink", "g")):
        if min(hidden, heads, kv_heads, dim, vdim) <= 0 or heads % kv_heads:
            raise ConfigError(f"Attention needs positive sizes and heads in whole groups, got heads={heads} kv_heads={kv_heads} "
                              f"dim={dim} vdim={vdim}.")
        if value_mix not in (None, "first", "blend"):
            raise ConfigError(f"value_mix must be None, 'first' or 'blend', got {value_mix!r}.")
        if softcap is not None and not softcap > 0:
            raise ConfigError(f"A cap on the scores must be positive, got {softcap!r}.")
        for name, n in (("mask_chunk", mask_chunk), ("window", window)):
            if n is not None and n <= 0:
                raise ConfigError(f"{name} must be positive, got {n!r}.")
        if sinks and sink_value is not None:
            raise ConfigError("The denominator's extra term is learned (sinks) or a constant (sink_value), not both.")
        if qkv_bias and head_gate:
            raise ConfigError("A gate per head rides in the q/k/v product, which then carries no biases.")
        rotary = getattr(position, "rotary_dim", 0)
        if rotary and (getattr(position, "pairing", None) != "halves" or rotary > dim or rotary % 2):
            raise ConfigError(f"This mixer turns the first {rotary} numbers of a head of {dim} in halves; the position "
                              f"encoding must pair them so and fit.")
        self.width = padded_width(dim, vdim)
        try:
            ops.check_attention_sizes(heads, kv_heads, self.width)
        except ops.KernelError as error:
            raise ConfigError(str(error)) from None
        self.hidden, self.heads, self.kv_heads, self.dim, self.vdim = hidden, heads, kv_heads, dim, vdim
        self.scale, self.position, self.qkv_bias, self.qk_norm, self.eps = float(scale), position, qkv_bias, qk_norm, float(eps)
        self.softcap, self.mask_chunk, self.window, self.sinks = softcap, mask_chunk, window, sinks
        self.value_mix, self.value_key, self.page_tokens = value_mix, value_key, page_tokens
        self.head_norm, self.sink_value, self.head_gate = bool(head_norm), sink_value, bool(head_gate)
        self.names = tuple(tensors) + ("g",) * (9 - len(tensors))

    # ------------------------------------------------------------------ what it keeps and costs
    def _reach(self):
        """How far back a query reads at most (None: to the start): what the cache may give back."""
        reaches = [n for n in (self.mask_chunk, self.window) if n is not None]
        return min(reaches) if reaches else None

    def cache_spec(self):
        return PagedKVSpec(self.kv_heads, self.width, self._reach(), self.page_tokens)

    def cache_elements_per_token(self) -> int:
        return 2 * self.kv_heads * self.width

    def flops(self, tokens: int, pairs: int = 0) -> float:
        q, k, v = self.heads * self.dim, self.kv_heads * self.dim, self.kv_heads * self.vdim
        projections = 2.0 * tokens * self.hidden * (q + k + v + (self.heads if self.head_gate else 0)) \
            + 2.0 * tokens * self.heads * self.vdim * self.hidden
        return projections + 2.0 * self.heads * (self.dim + self.vdim) * pairs

    def tensors(self):
        q, k, v, o, b, norm, blend, sink, gate = self.names
        H, G, D, V = self.heads, self.kv_heads, self.dim, self.vdim
        out = {q: TensorSpec((H * D, self.hidden)), k: TensorSpec((G * D, self.hidden)), v: TensorSpec((G * V, self.hidden)),
               o: TensorSpec((self.hidden, H * V))}
        if self.qkv_bias:
            out.update({q + b: TensorSpec((H * D,), "vector"), k + b: TensorSpec((G * D,), "vector"),
                        v + b: TensorSpec((G * V,), "vector")})
        if self.qk_norm:
            out.update({q + norm: TensorSpec((H * D,), "vector", "one_plus_normal"),
                        k + norm: TensorSpec((G * D,), "vector", "one_plus_normal")})
        if self.value_mix is not None:      # the first layer of a chain carries the number too, unused
            out[blend] = TensorSpec((), "vector")
        if self.sinks:
            out[sink] = TensorSpec((H,), "vector")
        if self.head_gate:
            out[gate] = TensorSpec((H, self.hidden))
        return out

    def bind(self, tensors):
        q, k, v, o, b, norm, blend, sink, gate = self.names
        self.w_qkv = torch.cat([tensors[q], tensors[k], tensors[v]] + ([tensors[gate]] if self.head_gate else []), dim=0).contiguous()
        self.gate_offset = (self.heads + self.kv_heads) * self.dim + self.kv_heads * self.vdim
        self.b_qkv = torch.cat([tensors[q + b], tensors[k + b], tensors[v + b]], dim=0).contiguous() if self.qkv_bias else None
        self.w_q_norm = tensors[q + norm] if self.qk_norm else None
        self.w_k_norm = tensors[k + norm] if self.qk_norm else None
        self.blend = tensors[blend].reshape(1).contiguous() if self.value_mix == "blend" else None
        self.sink = tensors[sink].to(torch.float32).contiguous() if self.sinks else None
        if self.sink_value is not None:
            self.sink = torch.full((self.heads,), float(self.sink_value), dtype=torch.float32, device=self.w_qkv.device)
        w_o = tensors[o]
        if self.width != self.vdim:      # columns of zeros where the cached values are wider than the values
            wide = torch.zeros(self.hidden, self.heads, self.width, dtype=w_o.dtype, device=w_o.device)
            wide[:, :, :self.vdim] = w_o.view(self.hidden, self.heads, self.vdim)
            w_o = wide.view(self.hidden, self.heads * self.width).contiguous()
        self.w_o = w_o
        self.w = {}

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def subparts(self):
        return [self.position]

    # ------------------------------------------------------------------ the step
    def forward(self, ctx, h, residual, cache):
        T, H, G, W = h.shape[0], self.heads, self.kv_heads, self.width
        proj = ctx.buffer("qkv", (T, self.w_qkv.shape[0]), ctx.act_dtype)
        ops.gemm(h, self.w_qkv, proj, bias=self.b_qkv)
        first = None
        if self.value_mix == "first":
            first = ctx.buffer(self.value_key, (T, G * self.vdim), ctx.act_dtype)
            ctx.shared[("values", self.value_key)] = first
        elif self.value_mix == "blend":
            first = ctx.shared.get(("values", self.value_key))
            if first is None or tuple(first.shape) != (T, G * self.vdim):
                raise ops.KernelError("A layer blends its values with an earlier layer's, but no earlier layer of this step has "
                                      "kept values of this shape.")
        queries = ctx.buffer("padded_q", (T, H * W), ctx.act_dtype)
        writes = cache.writes
        rotary = getattr(self.position, "rotary_dim", 0)
        ops.qkv_prepare(proj, H, G, self.dim, self.vdim, W, queries, positions=ctx.positions,
                        inv_freq=self.position.inv_freq if rotary else None,
                        inv_freq_tail=getattr(self.position, "inv_freq_tail", None) if rotary and proj.dtype == torch.float32 else None,
                        rotary_dim=rotary, q_norm=self.w_q_norm, k_norm=self.w_k_norm, eps=self.eps, blend=self.blend,
                        first=first, keep_first=self.value_mix == "first", slot_mapping=cache.slot_mapping if writes else None,
                        k_pool=cache.k if writes else None, v_pool=cache.v if writes else None,
                        magnitude=getattr(self.position, "magnitude", 1.0) if rotary else 1.0, head_norm=self.head_norm)
        mixed = ctx.buffer("attn", (T, H * W), ctx.act_dtype)
        project = None if self.head_gate else (self.w_o, residual)    # a gate stands between the heads' outputs and W_o
        if ops.attention(queries, H * W, cache.k, cache.v, cache.block_tables, ctx.attention, mixed, H, G, W, self.window,
                         self.scale, workspace=lambda n: ctx.buffer("attention_partials", (n,), torch.float32),
                         kind=ctx.attention_kind, project=project, scores="capped" if self.softcap else "scaled_dot",
                         softcap=self.softcap or 0.0, sinks=self.sink, mask_chunk=self.mask_chunk):
            return
        if self.head_gate:
            ops.head_gate(mixed, proj, self.gate_offset, H, W)
        ops.gemm(mixed, self.w_o, residual, accumulate=True)
