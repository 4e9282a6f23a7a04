"""Token embedding and output head (reference: src/qwen.ts:162-163, :203)."""
from __future__ import annotations

from .. import ops
from ..weights.loader import TensorSpec
from .base import Part, register_part


@register_part("embedding", "token_embedding")
class TokenEmbedding(Part):
    """x = table[token] * scale, float32."""

    graph_safe = True
    graph_safe_portions = True

    def __init__(self, vocab: int, hidden: int, tensor: str = "weight", scale: float = 1.0):
        self.vocab, self.hidden, self.tensor, self.scale = vocab, hidden, tensor, float(scale)

    def tensors(self):
        return {self.tensor: TensorSpec((self.vocab, self.hidden))}

    def forward(self, ctx, tokens, residual):
        ops.embed(self.w[self.tensor], tokens, residual)
        if self.scale != 1.0:
            ops.scale(residual, self.scale)

    def weight_elements(self) -> int:
        return 0      # a step gathers one row per token: nothing beside the matrices


@register_part("embedding", "bigram_embedding")
class BigramEmbedding(Part):
    """x = table[token] + pairs[(previous * mul_prev + token * mul_cur) mod buckets]; a sequence's first token takes
    the pair table's last row (row `buckets`).  The sum is float32.

    The token before a step's first token is part of a request's state: one int32 per request in a state slot,
    read and left behind by the kernel itself, so a step that is replayed from a graph with its tokens still on the
    device finds it too.  `tensors`: local names of the two tables."""

    graph_safe = True
    graph_safe_portions = True

    def __init__(self, vocab: int, hidden: int, buckets: int, mul_prev: int, mul_cur: int,
                 tensors: tuple = ("weight", "pairs.weight")):
        if buckets <= 0 or mul_prev < 0 or mul_cur < 0:
            raise ValueError(f"A pair table needs positive buckets and multipliers, got {buckets}, {mul_prev}, {mul_cur}.")
        self.vocab, self.hidden, self.buckets, self.mul_prev, self.mul_cur = vocab, hidden, buckets, mul_prev, mul_cur
        self.names = tuple(tensors)

    def tensors(self):
        return {self.names[0]: TensorSpec((self.vocab, self.hidden)),
                self.names[1]: TensorSpec((self.buckets + 1, self.hidden))}

    def cache_spec(self):
        from ..cache.spec import StateSpec
        return StateSpec((1,), "int32")

    def forward(self, ctx, tokens, residual, cache):
        ops.embed_bigram(self.w[self.names[0]], self.w[self.names[1]], tokens, ctx.positions, ctx.q_start, ctx.q_len,
                         ctx.seq_of_token, ctx.state_slots, cache.state, residual, ctx.n_seqs, self.buckets,
                         self.mul_prev, self.mul_cur)

    def weight_elements(self) -> int:
        return 0      # a step gathers two rows per token


@register_part("head", "linear_head")
class LinearHead(Part):
    """logits = (W . x) * scale in float32.  With `tied`, W is the embedding table and the head has no tensor."""

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, vocab: int, hidden: int, tied: bool, tensor: str = "weight", scale: float = 1.0):
        self.vocab, self.hidden, self.tied, self.tensor, self.scale = vocab, hidden, tied, tensor, float(scale)
        self.table = None

    def tensors(self):
        return {} if self.tied else {self.tensor: TensorSpec((self.vocab, self.hidden))}

    def bind(self, tensors):
        self.w = tensors
        if not self.tied:
            self.table = tensors[self.tensor]

    def tie(self, embedding_table):
        self.table = embedding_table

    def forward(self, ctx, h, logits):
        ops.gemm(h, self.table, logits)
        if self.scale != 1.0:
            ops.scale(logits, self.scale)

    def weight_elements(self) -> int:
        return self.vocab * self.hidden      # the output matrix is read whole, also where it is the embedding table

    def flops(self, tokens: int, pairs: int = 0) -> float:
        return 2.0 * tokens * self.vocab * self.hidden
