"""Plain Morarax forward pass: whole sequence, no cache, float64 arithmetic, one function per mechanism.

Shares no code with the engine.  `store` is an optional rounding function applied wherever the bfloat16 engine
keeps a tensor in bfloat16 (normed activations, projection outputs, the convolution's output, gated branches,
what enters an output projection); with the default (float32 rounding) everything is float32 storage over float64
sums.  What the design computes in 32 bits (angles, scores and weights, norms, gates and decays of a recurrence,
states, the residual sum) is never rounded by `store`.

Notation.  x: the residual stream [tokens, width].  Every layer has ONE norm: with h = rms(x) * w_norm,
x <- x + m * (ls1 * mixer(h) + ls2 * ff(h)), m the model's residual multiplier and ls1, ls2 vectors of the layer;
a layer may have no feed-forward.  Three mixers:
  "attention"  grouped-query softmax attention; the first rot.dims numbers of every head turn ("halves" pairing,
               frequencies optionally blended as in YaRN, cosine and sine scaled); after turning, every q and k head
               is divided by its root mean square; the softmax's denominator holds one extra 1 (a key of score 0
               without a value); head n's output is multiplied by sigmoid((W_g h)_n).
  "rglru"      two branches of `width` channels: y = gelu_tanh(W_y h + b_y) and u = conv(W_x h + b_x), a causal
               convolution per channel; gates r, i from block-diagonal matrices on u; a = exp(-8 r softplus(lam));
               S_t = a S_(t-1) + sqrt(1 - a^2) i u; output W_o (S * y).
  "retention"  per head S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t with turned q and k, k times dim^(-1/2);
               o divided by its root mean square per head, times silu(W_g h), then W_o.
Feed-forward: W_down (relu(W_gate h) * (W_up h)).  Logits: head (rms(x) * w_final) * logit_scale.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


def f32(x):
    return np.asarray(x, dtype=np.float64).astype(np.float32)


def bf16_round(x):
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(a.shape)


def read_safetensors(path: str) -> dict:
    """name -> float64 (or integer) array: 8 bytes of header length, the JSON header, then the data."""
    with open(path, "rb") as f:
        (n,) = struct.unpack("<Q", f.read(8))
        header = json.loads(f.read(n))
        data = f.read()
    out = {}
    for name, meta in header.items():
        if name == "__metadata__":
            continue
        lo, hi = meta["data_offsets"]
        raw = data[lo:hi]
        if meta["dtype"] == "BF16":
            a = (np.frombuffer(raw, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)
        elif meta["dtype"] == "F32":
            a = np.frombuffer(raw, dtype=np.float32).astype(np.float64)
        elif meta["dtype"] == "I32":
            a = np.frombuffer(raw, dtype=np.int32)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']}")
        out[name] = a.reshape(meta["shape"])
    return out


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ---------------------------------------------------------------------------------------------- small pieces
def sigmoid(z):
    z = np.asarray(z, dtype=np.float64)
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    z = np.asarray(z, dtype=np.float64)
    return z * sigmoid(z)


def softplus(z):
    z = np.asarray(z, dtype=np.float64)
    return np.logaddexp(0.0, z)


def gelu_tanh(z):
    z = np.asarray(z, dtype=np.float64)
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def linear(x, w, b=None):
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    return y if b is None else y + np.asarray(b, dtype=np.float64)


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt((x * x).mean(axis=-1, keepdims=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * np.asarray(weight, dtype=np.float64)


# ---------------------------------------------------------------------------------------------- positions
def pair_frequencies(rot: dict):
    """(frequency of every pair of turning numbers, factor on cosines and sines)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = np.arange(dims // 2, dtype=np.float64)
    freq = base ** (-2.0 * i / max(dims, 1))
    scaling = rot.get("scaling")
    if not scaling:
        return freq, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def dim_of(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return freq / factor * ramp + freq * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def turn_halves(x, positions, rot: dict):
    """x [tokens, heads, size]: number i of a head turns with number i + dims/2; numbers from `dims` on stay."""
    x = np.array(x, dtype=np.float64)
    dims = int(rot["dims"])
    half = dims // 2
    if half == 0:
        return x
    freq, magnitude = pair_frequencies(rot)
    angle = np.asarray(positions, dtype=np.float64)[:, None, None] * freq[None, None, :]
    c, s = np.cos(angle) * magnitude, np.sin(angle) * magnitude
    a, b = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = a * c - b * s
    x[..., half:dims] = b * c + a * s
    return x


# ---------------------------------------------------------------------------------------------- mixers
def softmax_plus_one(scores, allowed):
    """exp(s_j) / (1 + sum over allowed keys of exp(s_j))."""
    s = np.where(allowed, scores, -np.inf)
    top = np.maximum(s.max(axis=-1, keepdims=True), 0.0)
    e = np.exp(s - top)
    return e / (e.sum(axis=-1, keepdims=True) + np.exp(-top))


def attention_mixer(w, pre: str, m: dict, h, positions, eps: float, store=f32):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = store(linear(h, w[pre + "q"])).reshape(T, H, D)
    k = store(linear(h, w[pre + "k"])).reshape(T, G, D)
    v = store(linear(h, w[pre + "v"])).reshape(T, G, V)
    gate = sigmoid(store(linear(h, w[pre + "g"])))                      # [T, H]
    q = store(unit_rms(turn_halves(q, positions, m["rot"]), eps))
    k = store(unit_rms(turn_halves(k, positions, m["rot"]), eps))
    allowed = np.arange(T)[None, :] <= np.arange(T)[:, None]
    out = np.zeros((T, H, V))
    per = H // G
    for n in range(H):
        g = n // per
        scores = (q[:, n] @ k[:, g].T) * float(m["scale"])
        out[:, n] = softmax_plus_one(scores, allowed) @ v[:, g]
    out = store(store(out) * gate[:, :, None])
    return linear(out.reshape(T, H * V), w[pre + "o"])


def causal_conv(x, taps_weight, bias):
    """x [T, C], taps_weight [C, taps] (last column: the current token's), zeros before the start."""
    x = np.asarray(x, dtype=np.float64)
    kw = np.asarray(taps_weight, dtype=np.float64)
    T, C = x.shape
    taps = kw.shape[1]
    padded = np.concatenate([np.zeros((taps - 1, C)), x], axis=0)
    out = np.tile(np.asarray(bias, dtype=np.float64), (T, 1))
    for j in range(taps):
        out += padded[j:j + T] * kw[:, j][None, :]
    return out


def block_gate(u, weight, bias):
    """u [T, blocks * n] in `blocks` parts; part b goes through weight[b] [out, in] and bias[b]; sigmoid of the result."""
    weight = np.asarray(weight, dtype=np.float64)
    blocks, n, _ = weight.shape
    T = u.shape[0]
    parts = np.asarray(u, dtype=np.float64).reshape(T, blocks, n)
    z = np.einsum("tbi,boi->tbo", parts, weight) + np.asarray(bias, dtype=np.float64)[None]
    return sigmoid(z).reshape(T, blocks * n)


def gated_linear_recurrence(u, r, i, lam):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t from S = 0, a_t = exp(-8 r_t softplus(lam))."""
    a = np.exp(-8.0 * r * softplus(lam)[None, :])
    drive = np.sqrt(1.0 - a * a) * i * u
    out = np.zeros_like(drive)
    state = np.zeros(u.shape[1])
    for t in range(u.shape[0]):
        state = a[t] * state + drive[t]
        out[t] = state
    return out


def rglru_mixer(w, pre: str, m: dict, h, store=f32):
    y = store(gelu_tanh(store(linear(h, w[pre + "y"], w[pre + "y.b"]))))
    u = store(causal_conv(store(linear(h, w[pre + "x"], w[pre + "x.b"])), w[pre + "conv"], w[pre + "conv.b"]))
    r = block_gate(u, w[pre + "ra"], w[pre + "ra.b"])
    i = block_gate(u, w[pre + "ri"], w[pre + "ri.b"])
    states = gated_linear_recurrence(u, r, i, np.asarray(w[pre + "lam"], dtype=np.float64))
    return linear(store(states * y), w[pre + "o"])


def retention_mixer(w, pre: str, m: dict, h, positions, eps: float, store=f32):
    T = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = turn_halves(store(linear(h, w[pre + "q"])).reshape(T, H, D), positions, m["rot"])
    k = turn_halves(store(linear(h, w[pre + "k"])).reshape(T, H, D), positions, m["rot"]) * float(D) ** -0.5
    v = store(linear(h, w[pre + "v"])).reshape(T, H, V)
    gate = silu(store(linear(h, w[pre + "g"]))).reshape(T, H, V)
    out = np.zeros((T, H, V))
    for n in range(H):
        decay = float(m["decay"][n])
        state = np.zeros((D, V))
        for t in range(T):
            state = decay * state + np.outer(k[t, n], v[t, n])
            out[t, n] = state.T @ q[t, n]
    out = store(unit_rms(out, eps) * gate)
    return linear(out.reshape(T, H * V), w[pre + "o"])


def dense_ff(w, pre: str, h, store=f32):
    gate, up = store(linear(h, w[pre + "gate"])), store(linear(h, w[pre + "up"]))
    return linear(store(np.maximum(gate, 0.0) * up), w[pre + "down"])


# ---------------------------------------------------------------------------------------------- the model
def forward(w, cfg, tokens, store=f32, rows=None, streams=None):
    """Logits [len(rows) or T, vocab] of the whole sequence.  `streams`: a list that receives x after every layer."""
    eps = float(cfg["norm"]["eps"])
    mult = float(cfg["residual_mult"])
    x = np.asarray(w["embed"], dtype=np.float64)[np.asarray(tokens)]
    positions = np.arange(len(tokens))
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = store(rms_norm(x, w[pre + "norm1"], eps))
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            mixed = attention_mixer(w, pre + "mix.", m, h, positions, eps, store)
        elif kind == "rglru":
            mixed = rglru_mixer(w, pre + "mix.", m, h, store)
        elif kind == "retention":
            mixed = retention_mixer(w, pre + "mix.", m, h, positions, eps, store)
        else:
            raise ValueError(kind)
        total = mixed * np.asarray(w[pre + "ls1"], dtype=np.float64)
        if layer.get("mlp") is not None:
            total = total + dense_ff(w, pre + "mlp.", h, store) * np.asarray(w[pre + "ls2"], dtype=np.float64)
        x = x + mult * total
        if streams is not None:
            streams.append(x.copy())
    if rows is not None:
        x = x[np.asarray(rows)]
    x = store(rms_norm(x, w["final.norm"], eps))
    return (linear(x, w["head"]) * float(cfg["logit_scale"])).astype(np.float32)


def forward_logits(w, cfg, tokens, store=f32, rows=None):
    return forward(w, cfg, tokens, store=store, rows=rows)
