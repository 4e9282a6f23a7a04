"""Dense gated feed-forward (reference: src/qwen.ts:196-200)."""
from __future__ import annotations

import torch

from .. import ops
from ..weights.loader import TensorSpec
from .base import FeedForward, register_part


@register_part("feed_forward", "gated_mlp")
class GatedMLP(FeedForward):
    """down(act(gate(x), up(x))), no biases.  gate and up are kept as one matrix [2 * inner, hidden].  `activation`: one
    of `ops.GATE_ACTIVATIONS` ("silu": silu(g) * u; "clamped_swish": g' = min(g, limit), u' = clamp(u, -limit, limit),
    g' * sigmoid(1.702 g') * (u' + 1))."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, activation: str = "silu",
                 tensors: tuple = ("gate_proj.weight", "up_proj.weight", "down_proj.weight"), limit: float = 0.0):
        if activation not in ops.GATE_ACTIVATIONS:     # refused when the part is built, not at the first step
            raise ValueError(f"Gated feed-forward with activation {activation!r} has no kernel; "
                             f"there are kernels for {sorted(ops.GATE_ACTIVATIONS)}.")
        if activation == "clamped_swish" and not limit > 0:
            raise ValueError(f"The clamped activation needs a positive limit, got {limit!r}.")
        self.hidden, self.inner, self.activation, self.limit = hidden, inner, activation, float(limit)
        self.names = tuple(tensors)      # local names of the gate, up and down matrices

    def flops(self, tokens: int, pairs: int = 0) -> float:
        return 2.0 * tokens * 3 * self.hidden * self.inner

    def tensors(self):
        gate, up, down = self.names
        return {gate: TensorSpec((self.inner, self.hidden)), up: TensorSpec((self.inner, self.hidden)),
                down: TensorSpec((self.hidden, self.inner))}

    def bind(self, tensors):
        gate, up, down = self.names
        self.w_gate_up = torch.cat([tensors[gate], tensors[up]], dim=0).contiguous()
        self.w_down = tensors[down]
        self.w = {}

    def _fused(self, T: int, norm: bool) -> bool:
        return self.w_gate_up.dtype == torch.bfloat16 and ops.fused_supported(ops.FUSED_SILU, T, 2 * self.inner,
                                                                               self.hidden, norm=norm, variant=self.activation)

    fuse_input_norm = True    # see Attention.fuse_input_norm
    fuse_input_norm_f32 = True

    def forward_from_residual(self, ctx, norm, residual) -> bool:
        T = residual.shape[0]
        fold = norm.fold() if self.fuse_input_norm else None
        if fold is None or fold.kind != "rms":       # the one prologue the product kernels have
            return False
        if ctx.act_dtype == torch.float32 and self.fuse_input_norm_f32:
            act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
            if not ops.gate_up_silu_f32(self.w_gate_up, residual, act, activation=self.activation, norm_weight=fold.weight,
                                        eps=fold.eps, limit=self.limit):
                return False
            ops.gemm(act, self.w_down, residual, accumulate=True)
            return True
        if ctx.act_dtype != torch.bfloat16 or T > 64 or not self._fused(T, True):
            return False
        if not ops.fused_norm_pays(T, 2 * self.inner, self.hidden):
            return False
        act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
        ops.gate_up_silu(self.w_gate_up, act, residual=residual, norm_weight=fold.weight, eps=fold.eps,
                         activation=self.activation, limit=self.limit)
        ops.gemm(act, self.w_down, residual, accumulate=True)
        return True

    def forward(self, ctx, h, residual, row_gate=None, row_gate_column: int = 0):
        """`row_gate` (float32 [T, columns]): the token's output is multiplied by sigmoid(row_gate[t, row_gate_column]);
        the factor goes onto the gated product, of which the output is a linear function."""
        T = h.shape[0]
        act = ctx.buffer("gated", (T, self.inner), ctx.act_dtype)
        # (the older tiles, for a K in no whole steps of 64, have no epilogue for a row gate or another activation)
        plain = row_gate is None and self.activation == "silu"
        if ctx.act_dtype == torch.bfloat16 and self._fused(T, False) and (plain or T <= 64 or self.hidden % 64 == 0):
            ops.gate_up_silu(self.w_gate_up, act, x=h, activation=self.activation, limit=self.limit, row_gate=row_gate,
                             row_gate_column=row_gate_column)
        elif ctx.act_dtype == torch.float32 and ops.gate_up_silu_f32(
                self.w_gate_up, h, act, activation=self.activation, limit=self.limit, row_gate=row_gate,
                row_gate_column=row_gate_column):
            pass
        else:
            gu = ctx.buffer("gate_up", (T, 2 * self.inner), ctx.act_dtype)
            ops.gemm(h, self.w_gate_up, gu)
            ops.silu_mul(gu, act, activation=self.activation, limit=self.limit, row_gate=row_gate,
                         row_gate_column=row_gate_column)
        ops.gemm(act, self.w_down, residual, accumulate=True)


@register_part("feed_forward", "mlp")
class DenseMLP(FeedForward):
    """down(act(up(x) + b_up)) + b_down, no gate.  `activation`: one of `ops.UNARY_ACTIVATIONS` ("gelu_erf": the exact
    GELU, x * Phi(x)).  `bias`: the suffix of the biases' names, None for projections without them.  `tensors`: local
    names of the up and down matrices."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, activation: str = "gelu_erf", bias: str | None = ".b",
                 tensors: tuple = ("up", "down")):
        if activation not in ops.UNARY_ACTIVATIONS:
            raise ValueError(f"Feed-forward with activation {activation!r} has no kernel; there are kernels for "
                             f"{sorted(ops.UNARY_ACTIVATIONS)}.")
        self.hidden, self.inner, self.activation, self.bias = hidden, inner, activation, bias
        self.names = tuple(tensors)

    def flops(self, tokens: int, pairs: int = 0) -> float:
        return 2.0 * tokens * 2 * self.hidden * self.inner

    def tensors(self):
        up, down = self.names
        out = {up: TensorSpec((self.inner, self.hidden)), down: TensorSpec((self.hidden, self.inner))}
        if self.bias is not None:
            out.update({up + self.bias: TensorSpec((self.inner,), "vector"), down + self.bias: TensorSpec((self.hidden,), "vector")})
        return out

    def bind(self, tensors):
        up, down = self.names
        self.w_up, self.w_down = tensors[up], tensors[down]
        self.b_up = tensors[up + self.bias] if self.bias is not None else None
        self.b_down = tensors[down + self.bias] if self.bias is not None else None
        self.w = {}

    def forward_from_residual(self, ctx, norm, residual) -> bool:
        """A decode step's few tokens: the norm as the prologue of the up product, a launch less."""
        fold = norm.fold()
        if fold is None or fold.kind != "rms" or ctx.act_dtype != torch.bfloat16:
            return False
        T = residual.shape[0]
        act = ctx.buffer("mlp_inner", (T, self.inner), ctx.act_dtype)
        if not ops.gemm_from_residual(residual, fold.weight, fold.eps, self.w_up, act, bias=self.b_up):
            return False
        ops.activation(act, self.activation)
        ops.gemm(act, self.w_down, residual, bias=self.b_down, accumulate=True)
        return True

    def forward(self, ctx, h, residual):
        T = h.shape[0]
        act = ctx.buffer("mlp_inner", (T, self.inner), ctx.act_dtype)
        ops.gemm(h, self.w_up, act, bias=self.b_up)
        ops.activation(act, self.activation)
        ops.gemm(act, self.w_down, residual, bias=self.b_down, accumulate=True)
