"""A gated linear recurrence over channels behind a short causal convolution (the recurrent block of Griffin-like
designs): its memory is one float32 number per channel and request, and the convolution's last inputs."""
from __future__ import annotations

import torch

from .. import ops
from ..cache.spec import StateSpec
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import Mixer, register_part


@register_part("mixer", "gated_linear_recurrence")
class GatedLinearRecurrence(Mixer):
    """Two branches of `width` channels from the mixer's input h: y = gelu_tanh(W_y h + b_y) and u = conv(W_x h + b_x), a
    causal convolution of `taps` taps per channel (the last tap is the current token's; zeros before a request's first
    token).  The channels fall into `blocks` equal parts; part b has two square matrices [out, in] with biases:
    r = sigmoid(A_b u_b + a_b), i = sigmoid(I_b u_b + i_b).  Per channel a = exp(-rate * r * softplus(lam)) and
    S_t = a S_(t-1) + sqrt(1 - a^2) i u_t, from S = 0; the mixer's output is W_o (S * y).  `rate` is 8 in the kernel.

    Gates, decays and the state are float32.  What a request keeps between steps: S [width] and the convolution's last
    taps - 1 inputs, both float32 rows of fixed size, so requests of such a model share no prefix pages.

    `tensors`: local names of W_y, W_x, the convolution, the two gates' matrices, lam, W_o, and the biases' suffix.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, width: int, blocks: int, taps: int,
                 tensors: tuple = ("y", "x", "conv", "ra", "ri", "lam", "o", ".b")):
        if min(hidden, width, blocks, taps) <= 0 or width % blocks:
            raise ConfigError(f"A gated recurrence needs positive sizes and channels in equal parts, got width={width} "
                              f"blocks={blocks} taps={taps}.")
        self.hidden, self.width, self.blocks, self.taps = hidden, width, blocks, taps
        self.names = tuple(tensors)
        self._checked = False

    def cache_spec(self):
        spec = {"state": StateSpec((self.width,), "float32")}
        if self.taps > 1:
            spec["inputs"] = StateSpec((self.taps - 1, self.width), "float32")
        return spec

    def tensors(self):
        y, x, conv, ra, ri, lam, o, b = self.names
        W, n = self.width, self.width // self.blocks
        return {y: TensorSpec((W, self.hidden)), y + b: TensorSpec((W,), "vector"),
                x: TensorSpec((W, self.hidden)), x + b: TensorSpec((W,), "vector"),
                conv: TensorSpec((W, self.taps), "vector", "one_plus_normal"), conv + b: TensorSpec((W,), "vector"),
                ra: TensorSpec((self.blocks, n, n)), ra + b: TensorSpec((self.blocks, n), "vector"),
                ri: TensorSpec((self.blocks, n, n)), ri + b: TensorSpec((self.blocks, n), "vector"),
                lam: TensorSpec((W,), "vector", "one_plus_normal"), o: TensorSpec((self.hidden, W))}

    def flops(self, tokens: int, pairs: int = 0) -> float:
        n = self.width // self.blocks
        return 2.0 * tokens * (3 * self.hidden * self.width + 2 * self.width * n)

    def bind(self, tensors):
        y, x, conv, ra, ri, lam, o, b = self.names
        self.w_in = torch.cat([tensors[y], tensors[x]], dim=0).contiguous()
        self.b_in = torch.cat([tensors[y + b], tensors[x + b]], dim=0).contiguous()
        self.conv_w, self.conv_b = tensors[conv].contiguous(), tensors[conv + b].contiguous()
        # the gates' matrices input-major: neighbouring threads of the kernel own neighbouring outputs
        self.w_a, self.w_i = tensors[ra].transpose(1, 2).contiguous(), tensors[ri].transpose(1, 2).contiguous()
        self.b_a, self.b_i = tensors[ra + b].contiguous(), tensors[ri + b].contiguous()
        self.lam, self.w_o = tensors[lam].contiguous(), tensors[o]
        self.w = {}

    def forward(self, ctx, h, residual, cache):
        if not self._checked:
            if not ops.rglru_takes(self.width, self.blocks, self.taps):
                raise ops.KernelError(f"No kernel for a gated recurrence of width {self.width} in {self.blocks} parts with "
                                      f"{self.taps} taps.")
            self._checked = True
        T, W = h.shape[0], self.width
        proj = ctx.buffer("recurrence_in", (T, 2 * W), ctx.act_dtype)
        ops.gemm(h, self.w_in, proj, bias=self.b_in)
        scratch = ctx.buffer("recurrence_gates", (2, T, W), torch.float32)
        out = ctx.buffer("recurrence_out", (T, W), ctx.act_dtype)
        ops.rglru(proj, 0, W, W, self.blocks, self.taps, self.conv_w, self.conv_b, self.w_a, self.b_a, self.w_i, self.b_i,
                  self.lam, ctx.q_start, ctx.q_len, ctx.seq_of_token, ctx.state_slots, ctx.n_seqs, cache["state"].state,
                  cache["inputs"].state if self.taps > 1 else None, scratch[0], scratch[1], out, max_q_len=ctx.max_q_len,
                  workspace=lambda n: ctx.buffer("recurrence_carry", (n,), torch.float32))
        ops.gemm(out, self.w_o, residual, accumulate=True)
