"""State-space mixers: the state-space-duality form (one decay per head and token, a matrix state per head) and the
selective scan (one decay per channel, state and token).  Their memory is a float32 state of fixed size per request and
the last inputs of a short convolution."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import StateSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part
from .conv import ShortConv


@register_part("mixer", "state_space_duality")
class StateSpaceDuality(Mixer):
    """[z | u | B | C | dt] = W_in h with z, u of heads * vdim numbers, B, C of groups * state and dt of heads.  (u, B, C) pass
    a causal convolution of `taps` taps per channel with bias, then SiLU.  d = softplus(dt + dt_bias).  Head n (of group
    n // (heads / groups)) keeps S [state, vdim]: S_t = exp(-exp(A_log_n) d_t) S_(t-1) + d_t B_t u_t^T and
    y_t = S_t^T C_t + D_n u_t.  The heads' y, times silu(z), are RMS-normed in `norm_groups` equal parts (`eps` inside the
    root) times a weight, and W_o projects them.  Step sizes, decays, the state and the norm are float32.

    `tensors`: local names of W_in, the convolution and its bias, dt_bias, A_log, D, the norm's weight and W_o.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, heads: int, vdim: int, state: int, groups: int, taps: int, norm_groups: int, eps: float,
                 tensors: tuple = ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")):
        if min(hidden, heads, vdim, state, groups, taps, norm_groups) <= 0 or heads % groups or (heads * vdim) % norm_groups:
            raise ConfigError(f"A state-space-duality mixer needs heads in whole groups and a norm in equal parts, got heads={heads} "
                              f"groups={groups} vdim={vdim} norm_groups={norm_groups}.")
        if state > 256:
            raise ConfigError(f"The scan kernel holds a state of up to 256 rows a head, got {state}.")
        self.hidden, self.heads, self.vdim, self.state, self.groups, self.taps = hidden, heads, vdim, state, groups, taps
        self.norm_groups, self.eps = norm_groups, float(eps)
        self.inner = heads * vdim
        self.channels = self.inner + 2 * groups * state
        self.names = tuple(tensors)
        self.conv = ShortConv(self.channels, taps, tensor=self.names[1], bias=self.names[2], activation="silu")

    def cache_spec(self):
        spec = {"state": StateSpec((self.heads, self.state, self.vdim), "float32")}
        if self.taps > 1:
            spec["inputs"] = self.conv.cache_spec()
        return spec

    def tensors(self):
        w_in, _, _, dt_bias, a_log, skip, norm, o = self.names
        out = {w_in: TensorSpec((2 * self.inner + 2 * self.groups * self.state + self.heads, self.hidden)),
               dt_bias: TensorSpec((self.heads,), "vector"), a_log: TensorSpec((self.heads,), "vector"),
               skip: TensorSpec((self.heads,), "vector", "one_plus_normal"),
               norm: TensorSpec((self.inner,), "vector", "one_plus_normal"), o: TensorSpec((self.hidden, self.inner))}
        out.update(self.conv.tensors())
        return out

    def flops(self, tokens: int, pairs: int = 0) -> float:
        projections = 2.0 * tokens * self.hidden * (3 * self.inner + 2 * self.groups * self.state + self.heads)
        return projections + 4.0 * tokens * self.inner * self.state

    def bind(self, tensors):
        w_in, _, _, dt_bias, a_log, skip, norm, o = self.names
        self.w_in, self.w_o, self.w_norm = tensors[w_in], tensors[o], tensors[norm].contiguous()
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()
        self.dt_bias, self.a_log, self.skip = f32(dt_bias), f32(a_log), f32(skip)
        self.conv.bind({name: tensors[name] for name in self.conv.tensors()})
        self.w = {}

    def forward(self, ctx, h, residual, cache):
        T, inner = h.shape[0], self.inner
        proj = ctx.buffer("ssd_in", (T, self.w_in.shape[0]), ctx.act_dtype)
        ops.gemm(h, self.w_in, proj)
        xbc = ctx.buffer("ssd_conv", (T, self.channels), ctx.act_dtype)
        self.conv.forward(ctx, proj, xbc, cache.get("inputs"), x_off=inner)
        gated = ctx.buffer("ssd_gated", (T, inner), torch.float32)
        ops.ssd_scan(proj, 0, inner + self.channels, xbc, self.heads, self.vdim, self.state, self.groups, self.dt_bias,
                     self.a_log, self.skip, ctx.q_start, ctx.q_len, ctx.state_slots, ctx.n_seqs, cache["state"].state, gated,
                     max_q_len=ctx.max_q_len, workspace=lambda n: ctx.buffer("scan_chunks", (n,), torch.float32))
        normed = ctx.buffer("ssd_normed", (T, inner), ctx.act_dtype)
        ops.group_rmsnorm(gated, self.w_norm, self.eps, normed, self.norm_groups)
        ops.gemm(normed, self.w_o, residual, accumulate=True)


@register_part("mixer", "selective_scan")
class SelectiveScan(Mixer):
    """[u | z] = W_in h (inner numbers each); u passes a causal convolution of `taps` taps per channel with bias, then SiLU.
    r = W_r u (dt_rank numbers), [B | C] = W_bc u (state numbers each): the rows of one tensor W_x = [W_r; W_bc].
    d = softplus(W_dt r + b_dt), one per channel; A = -exp(A_log) [inner, state].  Channel c keeps S[c, :]:
    S_t[c, n] = exp(d_c A[c, n]) S_(t-1)[c, n] + d_c u_c B_n and y_c = S_t[c, :] . C + D_c u_c.  W_o projects y * silu(z).
    Step sizes (from the float32 result of W_dt on), decays and the state are float32.

    `tensors`: local names of W_in, the convolution and its bias, W_x, W_dt and its bias, A_log, D and W_o.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, state: int, dt_rank: int, taps: int,
                 tensors: tuple = ("in", "conv", "conv.b", "x", "dt", "dt.b", "A_log", "D", "o")):
        if min(hidden, inner, state, dt_rank, taps) <= 0:
            raise ConfigError(f"A selective scan needs positive sizes, got inner={inner} state={state} dt_rank={dt_rank} taps={taps}.")
        if state > 256:
            raise ConfigError(f"The scan kernel holds up to 256 states a channel, got {state}.")
        self.hidden, self.inner, self.state, self.dt_rank, self.taps = hidden, inner, state, dt_rank, taps
        self.names = tuple(tensors)
        self.conv = ShortConv(inner, taps, tensor=self.names[1], bias=self.names[2], activation="silu")

    def cache_spec(self):
        spec = {"state": StateSpec((self.inner, self.state), "float32")}
        if self.taps > 1:
            spec["inputs"] = self.conv.cache_spec()
        return spec

    def tensors(self):
        w_in, _, _, w_x, w_dt, b_dt, a_log, skip, o = self.names
        out = {w_in: TensorSpec((2 * self.inner, self.hidden)), w_x: TensorSpec((self.dt_rank + 2 * self.state, self.inner)),
               w_dt: TensorSpec((self.inner, self.dt_rank)), b_dt: TensorSpec((self.inner,), "vector"),
               a_log: TensorSpec((self.inner, self.state), "vector"), skip: TensorSpec((self.inner,), "vector", "one_plus_normal"),
               o: TensorSpec((self.hidden, self.inner))}
        out.update(self.conv.tensors())
        return out

    def flops(self, tokens: int, pairs: int = 0) -> float:
        projections = 2.0 * tokens * (3 * self.hidden * self.inner + self.inner * (2 * self.dt_rank + 2 * self.state))
        return projections + 4.0 * tokens * self.inner * self.state

    def bind(self, tensors):
        w_in, _, _, w_x, w_dt, b_dt, a_log, skip, o = self.names
        self.w_in, self.w_o, self.w_dt, self.b_dt = tensors[w_in], tensors[o], tensors[w_dt], tensors[b_dt]
        self.w_r = tensors[w_x][:self.dt_rank].contiguous()      # two products: the step sizes' input must lie by itself
        self.w_bc = tensors[w_x][self.dt_rank:].contiguous()
        self.rates = (-torch.exp(tensors[a_log].to(torch.float32))).contiguous()
        self.skip = tensors[skip].to(torch.float32).contiguous()
        self.conv.bind({name: tensors[name] for name in self.conv.tensors()})
        self.w = {}

    def forward(self, ctx, h, residual, cache):
        T, inner, N = h.shape[0], self.inner, self.state
        proj = ctx.buffer("scan_in", (T, 2 * inner), ctx.act_dtype)
        ops.gemm(h, self.w_in, proj)
        u = ctx.buffer("scan_conv", (T, inner), ctx.act_dtype)
        self.conv.forward(ctx, proj, u, cache.get("inputs"))
        low = ctx.buffer("scan_rank", (T, self.dt_rank), ctx.act_dtype)
        ops.gemm(u, self.w_r, low)
        bc = ctx.buffer("scan_bc", (T, 2 * N), ctx.act_dtype)
        ops.gemm(u, self.w_bc, bc)
        dt = ctx.buffer("scan_dt", (T, inner), torch.float32)
        ops.gemm(low, self.w_dt, dt, bias=self.b_dt)
        out = ctx.buffer("scan_out", (T, inner), ctx.act_dtype)
        ops.selective_scan(u, 0, proj, inner, dt, bc, 0, inner, N, self.rates, self.skip, ctx.q_start, ctx.q_len,
                           ctx.state_slots, ctx.n_seqs, cache["state"].state, out, max_q_len=ctx.max_q_len,
                           workspace=lambda n: ctx.buffer("scan_chunks", (n,), torch.float32))
        ops.gemm(out, self.w_o, residual, accumulate=True)
