"""Kodezen as a plan of parts.

Tensor names: `embed`, `final.norm`, `head`; layer i's start with `l<i>.`: `norm1`, `norm2`, `canon1` (the convolution of
the mixer's input); the mixer's under `mix.` (mamba2: `in`, `conv`, `conv.b`, `dt_bias`, `A_log`, `D`, `norm`, `o`; mamba1:
`in`, `conv`, `conv.b`, `x`, `dt`, `dt.b`, `A_log`, `D`, `o`; attention: `q`, `k`, `q.conv`, `k.conv`, `q.norm`, `k.norm`,
`talk`, `o`); the feed-forward's under `mlp.` (dense: `up`, `up.b`, `down`, `down.b`; routed: `router`, `e<n>.gate`,
`e<n>.up`, `e<n>.down`).
"""
from __future__ import annotations

from ..config.kodezen import KodezenConfig
from ..parts.base import make_part
from .plan import LayerCall, LayerPlan, ModelParts, ModelPlan, PartPlan

# The design gives no position limit; the engine's bookkeeping wants one.
MAX_POSITIONS = 1 << 22


def _norm(cfg: KodezenConfig, tensor: str, prefix: str = "") -> PartPlan:
    return PartPlan("norm", "rmsnorm", {"size": cfg.width, "eps": cfg.eps, "tensor": tensor, "one_plus": True}, prefix)


def _mixer(cfg: KodezenConfig, i: int, prefix: str) -> PartPlan:
    entry, W = cfg.layers[i], cfg.width
    m = entry.mixer
    if entry.kind == "mamba2":
        return PartPlan("mixer", "state_space_duality", {
            "hidden": W, "heads": m.heads, "vdim": m.vdim, "state": m.state, "groups": m.groups, "taps": m.conv,
            "norm_groups": m.norm_groups, "eps": cfg.eps}, prefix)
    if entry.kind == "mamba1":
        return PartPlan("mixer", "selective_scan", {"hidden": W, "inner": m.inner, "state": m.state, "dt_rank": m.dt_rank,
                                                    "taps": m.conv}, prefix)
    position = PartPlan("position", "rotary_interleaved", {"rotary_dim": m.rot_dims, "theta": m.rot_base}) if m.rot_dims \
        else PartPlan("position", "none", {"head_dim": m.dim})
    return PartPlan("mixer", "mixed_heads_attention", {
        "hidden": W, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "scale": m.scale, "position": position,
        "taps": m.conv, "eps": cfg.eps, "window": m.window, "keep_first": m.keep_first}, prefix)


def _feed_forward(cfg: KodezenConfig, i: int, prefix: str) -> PartPlan:
    ff = cfg.layers[i].ff
    if ff.kind == "dense":
        return PartPlan("feed_forward", "mlp", {"hidden": cfg.width, "inner": ff.ff, "activation": "gelu_erf", "bias": ".b"}, prefix)
    return PartPlan("feed_forward", "routed_experts", {
        "hidden": cfg.width, "inner": ff.ff, "experts": ff.experts, "top": ff.top, "router_bias": False, "activation": "silu",
        "routing": "sigmoid_top", "weight_on": "input"}, prefix)


def _layer(cfg: KodezenConfig, i: int) -> LayerPlan:
    base = f"l{i}."
    parts = {"mixer_norm": _norm(cfg, "norm1", base),
             "mixer_conv": PartPlan("conv", "short_conv", {"channels": cfg.width, "taps": cfg.canon_taps, "tensor": "canon1",
                                                           "residual": True}, base),
             "mixer": _mixer(cfg, i, base + "mix.")}
    if cfg.layers[i].ff is not None:
        parts["ffn_norm"] = _norm(cfg, "norm2", base)
        parts["ffn"] = _feed_forward(cfg, i, base + "mlp.")
    return LayerPlan("pre_norm", parts)


def _slots(layers: list) -> list:
    """One cache slot per thing a layer's parts keep (pages, states, a convolution's last inputs), numbered in the order in
    which the parts name them; what a part keeps is asked of the part itself."""
    schedule, free = [], 0
    for i, layer in enumerate(layers):
        block = make_part("block", layer.block, **{name: part.make() for name, part in layer.parts.items()})
        needs = ModelParts.cache_needs(block)
        schedule.append(LayerCall(i, {key: free + n for n, key in enumerate(needs)} or None))
        free += len(needs)
    return schedule


def build_kodezen(cfg: KodezenConfig) -> ModelPlan:
    layers = [_layer(cfg, i) for i in range(len(cfg.layers))]
    return ModelPlan(
        architecture=cfg.architecture, config=cfg, hidden_size=cfg.width, vocab_size=cfg.vocab, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding=PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": cfg.width,
                                                                              "tensor": "embed", "scale": cfg.embedding_scale}),
        layers=layers, schedule=_slots(layers), final_norm=_norm(cfg, "final.norm"),
        head=PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": cfg.width, "tied": False, "tensor": "head"}))
