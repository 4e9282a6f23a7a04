"""A feed-forward of routed experts, with an optional shared expert that every token takes."""
from __future__ import annotations

import torch

from .. import ops
from ..config.base import ConfigError
from ..weights.loader import TensorSpec
from .base import FeedForward, register_part
from .mlp import GatedMLP


@register_part("feed_forward", "routed_experts")
class RoutedExperts(FeedForward):
    """y = sum over a token's `top` experts of weight_e * down_e(act(gate_e x) * up_e x)  (+ shared(x)).

    Router logits z = W_r x + b are float32; the `top` largest are chosen (the lowest index wins a tie) and their
    weights are the softmax over the chosen logits alone.  Nothing is decided on the host: a kernel makes the choice,
    sorts the (token, choice) pairs by expert and cuts every expert's rows into tiles, the two grouped products walk those
    tiles (the first gathers its rows from the tokens and applies the activation, the second writes float32 rows),
    and the weighted sum is taken per token in the order of its choices, so a token's result does not depend on what
    else is in the step.

    hidden, inner, experts, top: sizes.  shared_inner: inner size of the shared expert (None: there is none).
    router_bias: whether the router has a bias.  `tensors`: local name patterns of an expert's gate, up and down
    matrices (`{e}` = the expert's number), of the router's weight and bias, and the prefix of the shared expert.

    routing "scored_groups" is another rule of choice: scores s = the softmax over ALL router outputs; the choice goes by
    s + correction (a tensor, `correction`) and only among the outputs of the `keep` best of `groups` equal groups of
    neighbours (a group's worth is its largest such sum); the weights are the chosen outputs' s times `route_scale`, not
    renormalised.  The last `identity` router outputs are experts without tensors that return their input.
    routing "sigmoid_top": the `top` largest logits are chosen and a choice's weight is the sigmoid of its logit, not
    renormalised.  weight_on "input": the weight multiplies what the expert reads, not what it returns: the output is the
    sum of expert_e(weight_e * x).
    activation / limit, shared_activation / shared_limit: see GatedMLP.  shared_gate: the local name of a [1, hidden]
    tensor g; the shared expert's output is then multiplied by sigmoid(g . x), one number per token.
    """

    graph_safe = True

    graph_safe_portions = True

    def __init__(self, hidden: int, inner: int, experts: int, top: int, shared_inner: int | None = None,
                 router_bias: bool = True, activation: str = "silu",
                 tensors: tuple = ("e{e}.gate", "e{e}.up", "e{e}.down", "router", "router.b", "shared."),
                 limit: float = 0.0, routing: str = "softmax_top", identity: int = 0, groups: int = 1, keep: int = 1,
                 route_scale: float = 1.0, correction: str | None = None, shared_activation: str | None = None,
                 shared_limit: float = 0.0, shared_gate: str | None = None, weight_on: str = "output"):
        if min(hidden, inner, experts, top) <= 0 or top > experts + identity or identity < 0:
            raise ConfigError(f"A routed feed-forward needs 0 < top <= experts and positive sizes, got top={top} "
                              f"experts={experts} inner={inner}.")
        if routing not in ("softmax_top", "scored_groups", "sigmoid_top"):
            raise ConfigError(f"No routing rule {routing!r}; there are 'softmax_top', 'sigmoid_top' and 'scored_groups'.")
        if weight_on not in ("output", "input") or (weight_on == "input" and identity):
            raise ConfigError(f"A choice's weight goes on the expert's 'output' or its 'input' (then without identity experts), got {weight_on!r}.")
        outputs = experts + identity
        if routing != "scored_groups" and (identity or groups != 1 or correction or route_scale != 1.0):
            raise ConfigError("Identity experts, groups, a correction and a scale belong to the rule 'scored_groups'.")
        if routing == "scored_groups":
            if groups <= 0 or outputs % groups or not 0 < keep <= groups or top > keep * (outputs // groups):
                raise ConfigError(f"{outputs} router outputs do not form {groups} equal groups of which {keep} hold {top} choices.")
            if outputs > 256:
                raise ConfigError(f"The grouped rule of choice takes up to 256 router outputs, got {outputs}.")
            if router_bias:
                raise ConfigError("The grouped rule of choice has a correction on the scores, not a bias on the logits.")
        if activation == "clamped_swish" and not limit > 0:
            raise ConfigError(f"The clamped activation needs a positive limit, got {limit!r}.")
        if activation not in ops.GATE_ACTIVATIONS:
            raise ConfigError(f"Experts with activation {activation!r} have no kernel; there are kernels for "
                              f"{sorted(ops.GATE_ACTIVATIONS)}.")
        self.hidden, self.inner, self.experts, self.top = hidden, inner, experts, top
        self.router_bias, self.activation, self.names = router_bias, activation, tuple(tensors)
        self.limit, self.routing, self.identity, self.groups, self.keep = float(limit), routing, identity, groups, keep
        self.route_scale, self.correction, self.shared_gate = float(route_scale), correction, shared_gate
        self.outputs, self.weight_on = outputs, weight_on
        prefix = self.names[5]
        try:
            self.shared = None if not shared_inner else GatedMLP(hidden, shared_inner, shared_activation or activation,
                                                                 tensors=(prefix + "gate", prefix + "up", prefix + "down"),
                                                                 limit=shared_limit if shared_activation else limit)
        except ValueError as error:
            raise ConfigError(str(error)) from None
        if shared_gate is not None and self.shared is None:
            raise ConfigError("A gate on the shared expert needs a shared expert.")

    def subparts(self):
        return [self.shared] if self.shared is not None else []

    def flops(self, tokens: int, pairs: int = 0) -> float:
        total = 2.0 * tokens * self.hidden * (self.outputs + 3 * self.inner * self.top)
        return total + (self.shared.flops(tokens) if self.shared is not None else 0.0)

    def tensors(self):
        gate, up, down, router, bias, _ = self.names
        out = {}
        for e in range(self.experts):
            out[gate.format(e=e)] = TensorSpec((self.inner, self.hidden))
            out[up.format(e=e)] = TensorSpec((self.inner, self.hidden))
            out[down.format(e=e)] = TensorSpec((self.hidden, self.inner))
        out[router] = TensorSpec((self.outputs, self.hidden))
        if self.router_bias:
            out[bias] = TensorSpec((self.experts,), "vector")
        if self.correction is not None:
            out[self.correction] = TensorSpec((self.outputs,), "vector")
        if self.shared is not None:
            out.update(self.shared.tensors())
        if self.shared_gate is not None:
            out[self.shared_gate] = TensorSpec((1, self.hidden))
        return out

    def bind(self, tensors):
        gate, up, down, router, bias, _ = self.names
        E = self.experts
        # [experts, 2 inner, hidden]: an expert's gate rows, then its up rows; [experts, hidden, inner]
        self.w_gate_up = torch.stack([torch.cat([tensors.pop(gate.format(e=e)), tensors.pop(up.format(e=e))], dim=0)
                                      for e in range(E)]).contiguous()
        self.w_down = torch.stack([tensors.pop(down.format(e=e)) for e in range(E)]).contiguous()
        self.w_router = tensors[router]
        if self.shared_gate is not None:      # the gate's one row rides behind the router's: one product for both
            self.w_router = torch.cat([self.w_router, tensors[self.shared_gate].reshape(1, self.hidden)], dim=0).contiguous()
        self.b_router = tensors[bias] if self.router_bias else None
        self.w_correction = tensors[self.correction].to(torch.float32).contiguous() if self.correction is not None else None
        if self.shared is not None:
            self.shared.bind({name: tensors[name] for name in self.shared.tensors()})
        self.w = {}

    def forward(self, ctx, h, residual):
        T, E, top = h.shape[0], self.experts, self.top
        pairs = T * top
        logits = ctx.buffer("router_logits", (T, self.w_router.shape[0]), torch.float32)
        ops.gemm(h, self.w_router, logits, bias=self.b_router)
        ids = ctx.buffer("expert_ids", (T, top), torch.int32)
        weights = ctx.buffer("expert_weights", (T, top), torch.float32)
        row_of_pair = ctx.buffer("expert_row_of_pair", (pairs,), torch.int32)
        pair_of_row = ctx.buffer("expert_pair_of_row", (pairs,), torch.int32)
        tile_rows = ops.group_tile_rows(ctx.act_dtype, pairs, E, self.hidden % 8 == 0 and self.inner % 8 == 0)
        tiles = ctx.buffer("expert_tiles", (3 * ops.route_max_tiles(pairs, E, tile_rows),), torch.int32)
        n_tiles = ctx.buffer("expert_tile_count", (1,), torch.int32)
        if self.routing == "scored_groups":
            ops.route_scored(logits, self.outputs, E, self.w_correction, self.groups, self.keep, self.route_scale, ids, weights,
                             row_of_pair, pair_of_row, tiles, n_tiles, tile_rows)
        elif self.routing == "sigmoid_top":
            ops.route_sigmoid(logits, ids, weights, row_of_pair, pair_of_row, tiles, n_tiles, tile_rows)
        else:
            ops.route(logits, ids, weights, row_of_pair, pair_of_row, tiles, n_tiles, tile_rows)
        act = ctx.buffer("expert_act", (pairs, self.inner), ctx.act_dtype)
        if self.weight_on == "input":      # every (token, choice) pair reads a row of its own: the token's, times the weight
            scaled = ctx.buffer("expert_in", (pairs, self.hidden), ctx.act_dtype)
            ops.scale_rows(h, weights, scaled)
            ops.expert_gate_up(scaled, self.w_gate_up, tiles, n_tiles, pair_of_row, 1, act, activation=self.activation,
                               tile_rows=tile_rows, limit=self.limit)
        else:
            ops.expert_gate_up(h, self.w_gate_up, tiles, n_tiles, pair_of_row, top, act, activation=self.activation,
                               tile_rows=tile_rows, limit=self.limit)
        out = ctx.buffer("expert_out", (pairs, self.hidden), torch.float32)
        ops.expert_down(act, self.w_down, tiles, n_tiles, out, tile_rows=tile_rows)
        if self.identity:      # a pair routed to an identity output has no row of `out`: the sum takes the token's input
            ops.route_combine_identity(out, row_of_pair, ids, weights, h, E, residual)
        else:
            ops.route_combine(out, row_of_pair, weights, residual, weighted=self.weight_on == "output")
        if self.shared is not None:
            if self.shared_gate is not None:
                self.shared.forward(ctx, h, residual, row_gate=logits, row_gate_column=self.outputs)
            else:
                self.shared.forward(ctx, h, residual)
