"""Tiny Morarax configurations, model folders with weights of the tests' own making, and the plain side's logits."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

from tests.plain import morarax_plain as M


def rot(dims, base=10000.0, scaling=None):
    out = {"dims": dims, "base": base}
    if scaling is not None:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def attention(heads, kv_heads, dim, vdim, scale, rotation):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                                           "rot": rotation}}


def rglru(width, blocks, conv):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}}


def retention(heads, dim, vdim, decay, rotation):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": rotation}}


def layer(mix, ff=None):
    out = copy.deepcopy(mix)
    out["mlp"] = None if ff is None else {"kind": "dense", "ff": ff}
    return out


def model(width, vocab, layers, eps=1e-5, mult=0.5, logit_scale=1.0):
    return {"architecture": "Morarax", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
            "logit_scale": logit_scale, "layers": layers}


# no size in whole eights or sixteens; heads that turn in part, not at all, and with blended frequencies; a convolution of
# four taps and of one; a layer without a feed-forward; a decay of 1 (nothing is forgotten) and one of 0.5
ODD = model(100, 77, [
    layer(retention(3, 20, 6, (0.5, 0.9, 1.0), rot(8, 300.0)), 28),
    layer(attention(6, 2, 12, 10, 0.4, rot(12, 50.0, (4.0, 16, 8.0, 2.0))), 36),
    layer(rglru(60, 3, 4)),
    layer(attention(3, 3, 20, 24, 0.05, rot(0)), 28),
    layer(rglru(36, 1, 1), 20),
    layer(retention(2, 10, 30, (0.97, 0.8), rot(0))),
], eps=1e-3, mult=0.8, logit_scale=1.7)
# sizes the matrix-core kernels take: keys narrower than values and wider, 16 query heads over one key/value head
GENERAL = model(128, 300, [
    layer(attention(4, 2, 32, 64, 0.2, rot(16)), 96),
    layer(rglru(192, 2, 3), 96),
    layer(retention(2, 32, 64, (0.9, 0.995), rot(32, 1000.0)), 64),
    layer(attention(16, 1, 64, 32, 0.1, rot(32, 250.0, (8.0, 64, 16.0, 1.0))), 96),
    layer(retention(4, 64, 16, (0.95, 0.99, 0.999, 0.9999), rot(16, 1e6))),
    layer(rglru(128, 8, 2), 32),
], mult=0.6, logit_scale=0.5)
# no attention at all: a model whose requests hold no pages, only state slots
STATES = model(64, 150, [
    layer(rglru(96, 4, 3), 64),
    layer(retention(4, 16, 32, (0.7, 0.9, 0.99, 0.999), rot(16, 500.0)), 48),
    layer(rglru(64, 2, 2)),
], mult=1.0, logit_scale=2.0)
# attention alone, every layer the same sizes
ATTENTION = model(96, 211, [
    layer(attention(6, 3, 16, 16, 0.25, rot(16, 100.0, (2.0, 32, 4.0, 1.0))), 64),
    layer(attention(6, 3, 16, 16, 0.25, rot(16, 100.0, (2.0, 32, 4.0, 1.0)))),
    layer(attention(2, 1, 48, 80, 0.15, rot(24)), 32),
], mult=0.7, logit_scale=1.0)

CONFIGS = {"odd": ODD, "general": GENERAL, "states": STATES, "attention": ATTENTION}
PAGE = {"odd": 16, "general": 16, "states": 8, "attention": 4}
SEED = {"odd": 24, "general": 25, "states": 26, "attention": 27}


def random_weights(cfg: dict, seed: int) -> dict:
    """name -> float32 array for every tensor the configuration needs (shapes asked from the engine's plan, values the
    tests' own): the table N(0, 1), matrices N(0, 0.08), the gates' square matrices N(0, 0.3), norm weights and layer
    scales 1 + N(0, 0.1), biases N(0, 0.2), convolutions N(0, 0.5), lam N(-1, 1)."""
    import sprout_lm_amd as S
    from sprout_lm_amd.registry import build_model_plan
    expected = build_model_plan(S.config_from_dict(cfg)).expected_tensors()
    rng = np.random.default_rng(seed)
    out = {}
    for name in sorted(expected):
        shape = tuple(expected[name].shape)
        last = name.split(".")[-1]
        if name == "embed":
            a = rng.normal(0.0, 1.0, shape)
        elif last in ("norm", "norm1", "ls1", "ls2"):
            a = 1.0 + rng.normal(0.0, 0.1, shape)
        elif last == "b":
            a = rng.normal(0.0, 0.2, shape)
        elif last == "conv":
            a = rng.normal(0.0, 0.5, shape)
        elif last == "lam":
            a = rng.normal(-1.0, 1.0, shape)
        elif last in ("ra", "ri"):
            a = rng.normal(0.0, 0.3, shape)
        else:
            a = rng.normal(0.0, 0.08, shape)
        out[name] = M.bf16_round(np.asarray(a, dtype=np.float32)).reshape(shape)
    return out


def write_folder(folder: str, cfg: dict, weights: dict) -> str:
    from sprout_lm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: torch.from_numpy(np.ascontiguousarray(a)).reshape(np.shape(a)).to(torch.bfloat16) for n, a in weights.items()})
    return folder


def make_folder(root: str, name: str) -> str:
    folder = os.path.join(root, "morarax_" + name)
    if not os.path.exists(os.path.join(folder, "model.safetensors")):
        write_folder(folder, CONFIGS[name], random_weights(CONFIGS[name], SEED[name]))
    return folder


_MODELS: dict = {}
_LOGITS: dict = {}


def plain_logits(folder: str, dtype: str, tokens) -> np.ndarray:
    """The plain implementation's logits at every position of `tokens`."""
    key = (folder, dtype, tuple(tokens))
    if key not in _LOGITS:
        if folder not in _MODELS:
            _MODELS[folder] = M.load_folder(folder)
        cfg, w = _MODELS[folder]
        _LOGITS[key] = M.forward(w, cfg, list(tokens), store=M.bf16_round if dtype == "bfloat16" else M.f32)
    return _LOGITS[key]


def tolerance(dtype: str, ref: np.ndarray) -> float:
    """Bound of |engine - plain| on a row of logits: float32 sums against float64 sums, or the bfloat16 roundings that
    the two sides make at nearly the same places."""
    return (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(np.abs(ref).max()))


def random_tokens(vocab: int, n: int, seed: int) -> list[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]
