"""Retention: linear attention with a fixed decay per head and no softmax; its memory is one float32 matrix per head and
request."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import StateSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part


@register_part("mixer", "retention")
class Retention(Mixer):
    """q = W_q h, k = W_k h (heads x dim), v = W_v h, g = W_g h (heads x vdim), no biases.  `position` (a rotary part with
    "halves" pairing) turns the first rotary_dim numbers of every q and k head; k is then multiplied by dim^(-1/2).  Per
    head, with decay d_h: S_t = d_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t (no softmax, no denominator).  Every head's o is
    divided by its root mean square (`eps` inside the root, no weight), the heads are multiplied by silu(g) and W_o
    projects them.  The state [heads, dim, vdim] per request is float32 and starts at zero.

    `tensors`: local names of W_q, W_k, W_v, W_g, W_o.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, dim: int, vdim: int, decay, eps: float, position,
                 tensors: tuple = ("q", "k", "v", "g", "o")):
        decay = tuple(float(d) for d in decay)
        if min(hidden, heads, dim, vdim) <= 0 or len(decay) != heads:
            raise ConfigError(f"Retention needs positive sizes and one decay per head, got heads={heads} dim={dim} vdim={vdim} "
                              f"and {len(decay)} decays.")
        if any(not 0.0 <= d <= 1.0 for d in decay):
            raise ConfigError(f"A head's decay lies in [0, 1], got {decay}.")
        rotary = getattr(position, "rotary_dim", 0)
        if rotary and (getattr(position, "pairing", None) != "halves" or rotary > dim or rotary % 2):
            raise ConfigError(f"This mixer turns the first {rotary} numbers of a head of {dim} in halves; the position "
                              f"encoding must pair them so and fit.")
        self.hidden, self.heads, self.dim, self.vdim, self.decay, self.eps = hidden, heads, dim, vdim, decay, float(eps)
        self.position = position
        self.names = tuple(tensors)
        self._checked = False

    def cache_spec(self):
        return StateSpec((self.heads, self.dim, self.vdim), "float32")

    def tensors(self):
        q, k, v, g, o = self.names
        H, D, V = self.heads, self.dim, self.vdim
        return {q: TensorSpec((H * D, self.hidden)), k: TensorSpec((H * D, self.hidden)), v: TensorSpec((H * V, self.hidden)),
                g: TensorSpec((H * V, self.hidden)), o: TensorSpec((self.hidden, H * V))}

    def flops(self, tokens: int, pairs: int = 0) -> float:
        H, D, V = self.heads, self.dim, self.vdim
        return 2.0 * tokens * self.hidden * (2 * H * D + 3 * H * V) + 4.0 * tokens * H * D * V

    def bind(self, tensors):
        q, k, v, g, o = self.names
        self.w_in = torch.cat([tensors[q], tensors[k], tensors[v], tensors[g]], dim=0).contiguous()
        self.w_o = tensors[o]
        self.decays = torch.tensor(self.decay, dtype=torch.float64).to(torch.float32).to(self.w_o.device)
        self.w = {}

    def prepare(self, device, dtype):
        self.position.prepare(device, dtype)

    def subparts(self):
        return [self.position]

    def forward(self, ctx, h, residual, cache):
        if not self._checked:
            if not ops.retention_takes(self.dim, self.vdim):
                raise ops.KernelError(f"No retention kernel for heads of {self.dim} and {self.vdim} numbers.")
            self._checked = True
        T, H, D, V = h.shape[0], self.heads, self.dim, self.vdim
        proj = ctx.buffer("retention_in", (T, self.w_in.shape[0]), ctx.act_dtype)
        ops.gemm(h, self.w_in, proj)
        rotary = getattr(self.position, "rotary_dim", 0)
        table = self.position.table(ctx) if rotary else None
        out = ctx.buffer("retention_out", (T, H * V), ctx.act_dtype)
        ops.retention(proj, 0, H * D, 2 * H * D, 2 * H * D + H * V, H, D, V, rotary, table, self.decays, self.eps,
                      ctx.q_start, ctx.q_len, ctx.state_slots, ctx.n_seqs, cache.state, out, max_q_len=ctx.max_q_len,
                      workspace=lambda n: ctx.buffer("retention_chunks", (n,), torch.float32))
        ops.gemm(out, self.w_o, residual, accumulate=True)
