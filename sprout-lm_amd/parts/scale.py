"""What stands between a sublayer's result and the residual stream."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorSpec
from .base import BranchScale, register_part


@register_part("scale", "layer_scale")
class LayerScale(BranchScale):
    """residual += multiplier * (w * branch), w a learned vector of `size` numbers (element by element) and `multiplier`
    a constant of the model.  `tensor`: the local name of w.  Two of them join the residual in one pass."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, size: int, multiplier: float = 1.0, tensor: str = "weight"):
        self.size, self.multiplier, self.tensor = size, float(multiplier), tensor

    def tensors(self):
        return {self.tensor: TensorSpec((self.size,), "vector", "one_plus_normal")}

    def add(self, ctx, residual, branch, other=None, other_branch=None):
        if other is None:
            ops.scaled_add(residual, branch, self.w[self.tensor], self.multiplier)
        else:
            ops.scaled_add(residual, branch, self.w[self.tensor], self.multiplier, other_branch, other.w[other.tensor],
                           other.multiplier)
