"""Learned norms: RMSNorm (reference: norm, src/qwen.ts:72-77) and layer norm, with or without bias."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorSpec
from .base import Norm, NormFold, register_part


@register_part("norm", "rmsnorm")
class RMSNorm(Norm):
    """y = x / sqrt(mean(x^2) + eps) * weight; sums in float32, the weight is used as it is.  `tensor`: the local
    name of the weight.  `one_plus`: the tensor holds the weight's distance from one, y = ... * (1 + tensor); the sum
    1 + tensor is taken once, in float32, when the tensor is bound."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, size: int, eps: float, tensor: str = "weight", one_plus: bool = False):
        self.size, self.eps, self.tensor, self.one_plus = size, eps, tensor, bool(one_plus)

    def tensors(self):
        return {self.tensor: TensorSpec((self.size,), "vector", "normal" if self.one_plus else "one_plus_normal")}

    def bind(self, tensors):
        self.w = tensors
        self.weight = tensors[self.tensor]
        if self.one_plus:
            import torch
            self.weight = (tensors[self.tensor].to(torch.float32) + 1.0).contiguous()

    def forward(self, ctx, x, out, rows=None):
        ops.rmsnorm(x, self.weight, self.eps, out, rows)
        return out

    def fold(self):
        return NormFold("rms", self.weight, self.eps)


@register_part("norm", "layernorm")
class LayerNorm(Norm):
    """y = (x - mean) / sqrt(mean((x - mean)^2) + eps) * weight (+ bias); sums in float32.  `tensor`: the local
    name of the weight (checkpoints that call a norm's weight by the norm's own name give the name here and the
    prefix up to it); `bias`: the local name of the bias, None for a norm without one."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, size: int, eps: float, tensor: str = "weight", bias: str | None = None):
        self.size, self.eps, self.tensor, self.bias = size, eps, tensor, bias

    def tensors(self):
        out = {self.tensor: TensorSpec((self.size,), "vector", "one_plus_normal")}
        if self.bias is not None:
            out[self.bias] = TensorSpec((self.size,), "vector")
        return out

    def _bias(self):
        return None if self.bias is None else self.w[self.bias]

    def forward(self, ctx, x, out, rows=None):
        ops.layernorm(x, self.w[self.tensor], self.eps, out, rows, bias=self._bias())
        return out

    def forward_pair(self, ctx, other, x, out, other_out) -> bool:
        """This norm and `other` of the same x in one pass, where `other` differs in its weight alone."""
        if not isinstance(other, LayerNorm) or other.size != self.size or other.eps != self.eps:
            return False
        ops.layernorm(x, self.w[self.tensor], self.eps, out, None, other.w[other.tensor], other_out, bias=self._bias(),
                      bias2=other._bias())
        return True
