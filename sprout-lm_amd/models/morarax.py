"""Morarax as a plan of parts.

Tensor names: `embed`, `final.norm`, `head`; layer i's start with `l<i>.`: `norm1`, the layer scales `ls1` (mixer) and
`ls2` (feed-forward); the mixer's under `mix.` (attention: `q`, `k`, `v`, `g`, `o`; rglru: `y`, `y.b`, `x`, `x.b`, `conv`,
`conv.b`, `ra`, `ra.b`, `ri`, `ri.b`, `lam`, `o`; retention: `q`, `k`, `v`, `g`, `o`); the feed-forward's under `mlp.`
(`gate`, `up`, `down`).
"""
from __future__ import annotations

from ..config.morarax import MoraraxConfig, Rotation
from .plan import LayerCall, LayerPlan, ModelPlan, PartPlan

# The design gives no position limit; the engine's bookkeeping wants one.
MAX_POSITIONS = 1 << 22


def _position(rot: Rotation, dim: int) -> PartPlan:
    if rot.dims == 0:
        return PartPlan("position", "none", {"head_dim": dim})
    return PartPlan("position", "rotary_neox", {"head_dim": dim, "theta": rot.base, "rotary_dim": rot.dims,
                                                "scaling": rot.scaling_dict()})


def _mixer(cfg: MoraraxConfig, i: int, prefix: str) -> PartPlan:
    entry, W = cfg.layers[i], cfg.width
    m = entry.mixer
    if entry.kind == "attention":
        # the softmax's denominator holds one more 1: a constant logit of 0 without key or value
        return PartPlan("mixer", "sink_attention", {
            "hidden": W, "heads": m.heads, "kv_heads": m.kv_heads, "dim": m.dim, "vdim": m.vdim, "scale": m.scale,
            "position": _position(m.rot, m.dim), "eps": cfg.eps, "sinks": False, "sink_value": 0.0, "head_norm": True,
            "head_gate": True}, prefix)
    if entry.kind == "rglru":
        return PartPlan("mixer", "gated_linear_recurrence", {"hidden": W, "width": m.width, "blocks": m.blocks,
                                                             "taps": m.conv}, prefix)
    return PartPlan("mixer", "retention", {"hidden": W, "heads": m.heads, "dim": m.dim, "vdim": m.vdim, "decay": m.decay,
                                           "eps": cfg.eps, "position": _position(m.rot, m.dim)}, prefix)


def _layer(cfg: MoraraxConfig, i: int) -> LayerPlan:
    entry, base, W = cfg.layers[i], f"l{i}.", cfg.width
    scale = lambda name: PartPlan("scale", "layer_scale", {"size": W, "multiplier": cfg.residual_mult, "tensor": name}, base)
    parts = {"mixer_norm": PartPlan("norm", "rmsnorm", {"size": W, "eps": cfg.eps, "tensor": "norm1"}, base),
             "mixer": _mixer(cfg, i, base + "mix."), "mixer_scale": scale("ls1")}
    if entry.ff is not None:
        parts["ffn"] = PartPlan("feed_forward", "gated_mlp", {"hidden": W, "inner": entry.ff, "activation": "relu",
                                                              "tensors": ("gate", "up", "down")}, base + "mlp.")
        parts["ffn_scale"] = scale("ls2")
    return LayerPlan("parallel_scaled", parts)


def _slots(cfg: MoraraxConfig) -> list:
    """One cache slot per thing a layer's mixer keeps: pages for attention, one state for retention, the state and (with
    more than one tap) the convolution's inputs for the recurrence."""
    schedule, free = [], 0
    for i, layer in enumerate(cfg.layers):
        if layer.kind == "rglru" and layer.mixer.conv > 1:
            schedule.append(LayerCall(i, {"mixer.state": free, "mixer.inputs": free + 1}))
            free += 2
        elif layer.kind == "rglru":
            schedule.append(LayerCall(i, {"mixer.state": free}))
            free += 1
        else:
            schedule.append(LayerCall(i, free))
            free += 1
    return schedule


def build_morarax(cfg: MoraraxConfig) -> ModelPlan:
    W = cfg.width
    return ModelPlan(
        architecture=cfg.architecture, config=cfg, hidden_size=W, vocab_size=cfg.vocab, max_positions=MAX_POSITIONS,
        eos_token_ids=(), embedding=PartPlan("embedding", "token_embedding", {"vocab": cfg.vocab, "hidden": W, "tensor": "embed"}),
        layers=[_layer(cfg, i) for i in range(len(cfg.layers))], schedule=_slots(cfg),
        final_norm=PartPlan("norm", "rmsnorm", {"size": W, "eps": cfg.eps, "tensor": "final.norm"}),
        head=PartPlan("head", "linear_head", {"vocab": cfg.vocab, "hidden": W, "tied": False, "tensor": "head",
                                              "scale": cfg.logit_scale}))
