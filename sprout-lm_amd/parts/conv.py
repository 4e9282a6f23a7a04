"""A short causal convolution over time on every channel, as a part of its own: it keeps a request's last inputs."""
from __future__ import annotations

from .. import ops
from ..cache.spec import StateSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Part, register_part


@register_part("conv", "short_conv")
class ShortConv(Part):
    """y_t = act(b + sum_j w[:, j] * x_(t - taps + 1 + j)) (+ x_t with `residual`), per channel, zeros before a request's
    first token; the last tap is the current token's.  What a request keeps between steps: its last taps - 1 inputs,
    float32 [taps - 1, channels] (nothing with one tap).  `tensor`: the local name of w [channels, taps]; `bias`: the local
    name of b, None for a convolution without one; `activation`: None or "silu"."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, channels: int, taps: int, tensor: str = "conv", bias: str | None = None, residual: bool = False,
                 activation: str | None = None):
        if channels <= 0 or not 0 < taps <= 64:
            raise ConfigError(f"A short convolution needs channels and 1 to 64 taps, got {channels} and {taps}.")
        if activation not in (None, "silu"):
            raise ConfigError(f"A short convolution is followed by nothing or by 'silu', not {activation!r}.")
        self.channels, self.taps, self.tensor, self.bias = channels, taps, tensor, bias
        self.residual, self.activation = bool(residual), activation

    def tensors(self):
        out = {self.tensor: TensorSpec((self.channels, self.taps), "vector")}
        if self.bias is not None:
            out[self.bias] = TensorSpec((self.channels,), "vector")
        return out

    def cache_spec(self):
        return StateSpec((self.taps - 1, self.channels), "float32") if self.taps > 1 else None

    def bind(self, tensors):
        self.w = tensors
        self.weight = tensors[self.tensor].t().contiguous()      # tap-major: neighbouring channels lie together
        self.b = tensors[self.bias].contiguous() if self.bias is not None else None

    def forward(self, ctx, x, out, cache, x_off: int = 0, out_off: int = 0):
        """out[:, out_off : out_off + channels] = conv(x[:, x_off : x_off + channels]); x and out are different tensors."""
        ops.short_conv(x, x_off, self.channels, self.taps, self.weight, self.b, out, out_off, ctx.q_start, ctx.q_len,
                       ctx.seq_of_token, ctx.state_slots, ctx.n_seqs, cache.state if self.taps > 1 else None,
                       act=self.activation, add_input=self.residual, max_q_len=ctx.max_q_len)
        return out
