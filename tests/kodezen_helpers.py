"""Tiny Kodezen configurations, model folders with weights of the tests' own making, and the plain side's logits."""
from __future__ import annotations

import copy
import json
import os

import numpy as np
import torch

from tests.plain import kodezen_plain as K


def mamba2(heads, vdim, state, groups, conv, norm_groups):
    return {"type": "mamba2", "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                                        "norm_groups": norm_groups}}


def mamba1(inner, state, dt_rank, conv):
    return {"type": "mamba1", "mixer": {"inner": inner, "state": state, "dt_rank": dt_rank, "conv": conv}}


def attention(heads, kv_heads, dim, scale, conv, rot_dims, rot_base=10000.0, mask=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "conv": conv,
             "rot": {"dims": rot_dims, "base": rot_base}}
    if mask is not None:
        mixer["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return {"type": "attention", "mixer": mixer}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(mix, ff=None):
    out = copy.deepcopy(mix)
    out["mlp"] = ff
    return out


def model(width, vocab, layers, eps=1e-5, scale=4.0, taps=4):
    return {"architecture": "Kodezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "embedding": {"scale": scale},
            "canon": {"taps": taps}, "layers": layers}


# no size in whole eights; a state of five rows and of one; a window of seven keys that keeps two; every head a key/value
# head of its own; heads that turn in part and not at all; convolutions of one tap; a layer without feed-forward; every
# expert chosen
ODD = model(100, 77, [
    layer(mamba2(3, 10, 5, 1, 2, 3), moe(5, 2, 12)),
    layer(attention(6, 3, 12, 0.4, 3, 8, 50.0, (7, 2)), dense(28)),
    layer(mamba1(36, 5, 3, 4), dense(20)),
    layer(attention(3, 3, 20, 0.05, 1, 0)),
    layer(mamba2(4, 6, 9, 2, 1, 1), moe(3, 3, 10)),
    layer(mamba1(20, 1, 1, 1), dense(12)),
], eps=1e-3, scale=3.0, taps=3)
# sizes the matrix-core kernels take: one key/value head under four, four under eight; more kept keys than a page holds;
# a window without kept keys; states of 64 and 128 rows
GENERAL = model(128, 300, [
    layer(attention(4, 1, 32, 0.2, 4, 32, 1000.0, (24, 20)), dense(96)),
    layer(mamba2(4, 32, 64, 1, 4, 2), moe(4, 1, 64)),
    layer(mamba1(256, 16, 8, 4), dense(64)),
    layer(attention(8, 4, 16, 0.3, 2, 8, 250.0, (64, 0)), moe(8, 2, 32)),
    layer(mamba2(8, 16, 128, 4, 3, 4)),
], scale=8.0, taps=4)
# no attention at all: a model whose requests hold no pages, only state slots; the input convolution has one tap
STATES = model(64, 150, [
    layer(mamba1(96, 12, 4, 3), dense(64)),
    layer(mamba2(4, 16, 16, 2, 2, 1), dense(48)),
    layer(mamba1(64, 40, 16, 2)),
], scale=1.0, taps=1)
# attention alone: a window of one key, kept keys that fill a page exactly, no window
ATTENTION = model(96, 211, [
    layer(attention(6, 3, 16, 0.25, 2, 16, 100.0, (1, 0)), dense(64)),
    layer(attention(6, 2, 16, 0.25, 3, 4, 100.0, (9, 4)), moe(4, 2, 24)),
    layer(attention(2, 1, 48, 0.15, 1, 24), dense(32)),
], scale=2.0, taps=2)

CONFIGS = {"odd": ODD, "general": GENERAL, "states": STATES, "attention": ATTENTION}
PAGE = {"odd": 16, "general": 16, "states": 8, "attention": 4}
SEED = {"odd": 34, "general": 35, "states": 36, "attention": 37}


def random_array(rng, name: str, shape) -> np.ndarray:
    """Values for the tensor `name` by the last pieces of its name: the table N(0, 1), matrices N(0, 0.08), the small
    matrices of the scans N(0, 1 / inputs), the router wider, norm weights around zero or one as the design stores them, biases N(0, 0.2),
    convolutions N(0, 0.5), step-size biases N(-1, 1), logarithms of rates N(0, 0.7), the mixing matrix I + N(0, 0.3)."""
    last = name.split(".")[-1]
    if name == "embed":
        return rng.normal(0.0, 1.0, shape)
    if last in ("norm1", "norm2") or name == "final.norm":
        return rng.normal(0.0, 0.1, shape)
    if last in ("norm", "D"):
        return 1.0 + rng.normal(0.0, 0.1, shape)
    if name.endswith("dt.b") or last == "dt_bias":
        return rng.normal(-1.0, 1.0, shape)
    if last == "b":
        return rng.normal(0.0, 0.2, shape)
    if last in ("conv", "canon1"):
        return rng.normal(0.0, 0.5, shape)
    if last == "A_log":
        return rng.normal(0.0, 0.7, shape)
    if last == "talk":
        return np.eye(shape[0]) + rng.normal(0.0, 0.3, shape)
    if last in ("x", "dt"):
        return rng.normal(0.0, 1.0 / np.sqrt(shape[1]), shape)
    if last == "router":
        return rng.normal(0.0, 0.6, shape)
    return rng.normal(0.0, 0.08, shape)


def random_weights(cfg: dict, seed: int) -> dict:
    """name -> float32 array for every tensor the configuration needs (shapes asked from the engine's plan, values the
    tests' own), rounded to what bfloat16 holds."""
    import sprout_lm_amd as S
    from sprout_lm_amd.registry import build_model_plan
    expected = build_model_plan(S.config_from_dict(cfg)).expected_tensors()
    rng = np.random.default_rng(seed)
    out = {}
    for name in sorted(expected):
        shape = tuple(expected[name].shape)
        out[name] = K.bf16_round(np.asarray(random_array(rng, name, shape), dtype=np.float32)).reshape(shape)
    return out


def write_folder(folder: str, cfg: dict, weights: dict) -> str:
    from sprout_lm_amd.weights.safetensors_io import write_safetensors
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f, indent=1)
    write_safetensors(os.path.join(folder, "model.safetensors"),
                      {n: torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).reshape(np.shape(a)).to(torch.bfloat16)
                       for n, a in weights.items()})
    return folder


def make_folder(root: str, name: str) -> str:
    folder = os.path.join(root, "kodezen_" + name)
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
            _MODELS[folder] = K.load_folder(folder)
        cfg, w = _MODELS[folder]
        _LOGITS[key] = K.forward(w, cfg, list(tokens), store=K.bf16_round if dtype == "bfloat16" else K.f32)
    return _LOGITS[key]


def tolerance(dtype: str, ref: np.ndarray) -> float:
    """Bound of |engine - plain| on a row of logits: float32 sums against float64 sums, or the bfloat16 roundings that
    the two sides make at nearly the same places."""
    return (2e-5 if dtype == "float32" else 3e-2) * max(1.0, float(np.abs(ref).max()))


def random_tokens(vocab: int, n: int, seed: int) -> list[int]:
    return [int(t) for t in np.random.default_rng(seed).integers(0, vocab, n)]
