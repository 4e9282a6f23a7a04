"""Plain Kodezen forward pass: whole sequence, no cache, float64 arithmetic, one function per mechanism.

Shares no code with the engine.  `store` is an optional rounding function applied wherever the bfloat16 engine keeps a
tensor in bfloat16 (normed activations, projection outputs, what enters an output projection); with the default
(float32 rounding) everything is float32 storage over float64 sums.  What the design computes in 32 bits (angles,
scores and weights, norms, router scores, decays, step sizes and states of the recurrences, the residual sum) is never
rounded by `store`.

Notation.  x: the residual stream [tokens, width], x0 = embed[token] * embedding.scale.  A layer is
  h = n1(x);  h <- h + conv_c(h);  x <- x + mixer(h);  x <- x + ff(n2(x))        (the feed-forward may be absent)
with n(x) = x / sqrt(mean(x^2) + eps) * (1 + w) and conv_c a causal convolution over time per channel (`canon.taps` taps,
the last tap the current token's, zeros before the sequence).  Three mixers:
  "mamba2"     [z | u | B | C | dt] = W_in h; (u, B, C) pass a causal convolution with bias and silu; d = softplus(dt +
               dt_bias); per head n (group g(n)): S_t = exp(-exp(A_log_n) d_t) S_(t-1) + d_t B_t u_t^T, y_t = S_t^T C_t +
               D_n u_t; y * silu(z), RMS norm in `norm_groups` parts times a weight, W_o.
  "mamba1"     [u | z] = W_in h; u passes a causal convolution with bias and silu; [r | B | C] = W_x u; d = softplus(W_dt
               r + b); per channel c: S_t[c, :] = exp(d_c A[c, :]) S_(t-1)[c, :] + d_c u_c B_t, y_c = S_t[c, :] . C_t +
               D_c u_c; y * silu(z), W_o.
  "attention"  q = conv(W_q h), k = conv(W_k h) (a short causal convolution per channel, no bias); the values are k as it
               leaves the convolution; q and k are RMS-normed per head with a shared weight of size dim and the first
               rot.dims numbers of every head turn (pairs 2i, 2i + 1); position i sees j <= i with i - j < mask.size or
               j < mask.keep_first; ordinary softmax; the heads' weights are mixed by a matrix T [heads, heads] after
               the softmax, and head n applies its mixed weights to the values of its own key/value head; W_o.
Feed-forwards: dense W_down gelu_erf(W_up h + b) + b, or routed experts: s = sigmoid(W_r h), the `top` largest are chosen,
and the output is the sum over the chosen e of expert_e(s_e h), expert(v) = W_down(silu(W_gate v) * (W_up v)).
Logits: head n(x) with the final norm's weight.
"""
from __future__ import annotations

import json
import math
import os
import struct

import numpy as np


def f32(x):
    return np.asarray(x, dtype=np.float64).astype(np.float32).astype(np.float64)


def bf16_round(x):
    a = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    bits = a.view(np.uint32).astype(np.uint64)
    rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16
    return rounded.astype(np.uint32).view(np.float32).reshape(a.shape).astype(np.float64)


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
            a = np.frombuffer(raw, dtype=np.int32).astype(np.int64)
        else:
            raise ValueError(f"{name}: dtype {meta['dtype']} is not read here")
        out[name] = a.reshape(meta["shape"])
    return out


def load_folder(folder: str):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    return cfg, read_safetensors(os.path.join(folder, "model.safetensors"))


# ---------------------------------------------------------------------------------------------- small functions
def linear(x, w, b=None):
    y = np.asarray(x, dtype=np.float64) @ np.asarray(w, dtype=np.float64).T
    return y if b is None else y + np.asarray(b, dtype=np.float64)


def silu(x):
    return x / (1.0 + np.exp(-x))


def softplus(x):
    return np.logaddexp(0.0, x)


_erf = np.vectorize(math.erf, otypes=[np.float64])


def gelu_erf(x):
    return 0.5 * x * (1.0 + _erf(x / math.sqrt(2.0)))


def rms(x, eps):
    """x divided by its root mean square over the last axis, eps inside the root."""
    x = np.asarray(x, dtype=np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def one_plus_norm(x, w, eps):
    return rms(x, eps) * (1.0 + np.asarray(w, dtype=np.float64))


def causal_conv(u, w, b=None):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token.  u [T, channels], w [channels, taps]."""
    u, w = np.asarray(u, dtype=np.float64), np.asarray(w, dtype=np.float64)
    T, taps = u.shape[0], w.shape[1]
    y = np.zeros_like(u)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            y[back:] += u[:T - back] * w[:, j]
    return y if b is None else y + np.asarray(b, dtype=np.float64)


def turn_pairs(x, positions, dims: int, base: float):
    """Rotary positions on the first `dims` numbers of the last axis, number 2i with number 2i + 1; x [T, heads, dim]."""
    out = np.array(x, dtype=np.float64)
    if dims == 0:
        return out
    i = np.arange(dims // 2)
    angle = np.asarray(positions, dtype=np.float64)[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    a, b = out[..., 0:dims:2].copy(), out[..., 1:dims:2].copy()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def visible(T: int, size: int, keep_first: int):
    """[T, T] mask: query i sees key j."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


# ---------------------------------------------------------------------------------------------- mixers
def attention_mixer(w, pre: str, m, h, positions, eps, store=f32):
    T = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    V = m["vdim"]
    q = store(causal_conv(store(linear(h, w[pre + "q"])), w[pre + "q.conv"])).reshape(T, H, D)
    k = store(causal_conv(store(linear(h, w[pre + "k"])), w[pre + "k.conv"])).reshape(T, G, D)
    values = k[..., :V]
    qn = store(rms(q, eps) * np.asarray(w[pre + "q.norm"], dtype=np.float64))
    kn = store(rms(k, eps) * np.asarray(w[pre + "k.norm"], dtype=np.float64))
    qn = store(turn_pairs(qn, positions, m["rot"]["dims"], m["rot"]["base"]))
    kn = store(turn_pairs(kn, positions, m["rot"]["dims"], m["rot"]["base"]))
    mask = visible(T, m["mask"]["size"], m["mask"]["keep_first"]) if m.get("mask") else visible(T, T + 1, 0)
    weights = np.zeros((H, T, T))
    for n in range(H):
        s = (qn[:, n] @ kn[:, n // (H // G)].T) * float(m["scale"])
        s = np.where(mask, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        weights[n] = e / e.sum(axis=1, keepdims=True)
    mixed = np.einsum("ng,gij->nij", np.asarray(w[pre + "talk"], dtype=np.float64), weights)
    out = np.zeros((T, H, V))
    for n in range(H):
        out[:, n] = mixed[n] @ values[:, n // (H // G)]
    return linear(store(out.reshape(T, H * V)), w[pre + "o"])


def mamba2_mixer(w, pre: str, m, h, eps, store=f32):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    proj = store(linear(h, w[pre + "in"]))
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = store(silu(causal_conv(xbc, w[pre + "conv"], w[pre + "conv.b"])))
    u = xbc[:, :inner].reshape(T, H, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    d = softplus(dt + np.asarray(w[pre + "dt_bias"], dtype=np.float64))            # [T, H]
    rate = np.exp(np.asarray(w[pre + "A_log"], dtype=np.float64))
    skip = np.asarray(w[pre + "D"], dtype=np.float64)
    y = np.zeros((T, H, P))
    for n in range(H):
        g = n // (H // G)
        state = np.zeros((N, P))
        for t in range(T):
            state = math.exp(-rate[n] * d[t, n]) * state + d[t, n] * np.outer(B[t, g], u[t, n])
            y[t, n] = state.T @ C[t, g] + skip[n] * u[t, n]
    y = y.reshape(T, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * np.asarray(w[pre + "norm"], dtype=np.float64)
    return linear(store(y), w[pre + "o"])


def mamba1_mixer(w, pre: str, m, h, store=f32):
    T = h.shape[0]
    inner, N, R = m["inner"], m["state"], m["dt_rank"]
    proj = store(linear(h, w[pre + "in"]))
    u, z = proj[:, :inner], proj[:, inner:]
    u = store(silu(causal_conv(u, w[pre + "conv"], w[pre + "conv.b"])))
    low = store(linear(u, w[pre + "x"]))
    r, B, C = low[:, :R], low[:, R:R + N], low[:, R + N:]
    d = softplus(linear(r, w[pre + "dt"], w[pre + "dt.b"]))                        # [T, inner]
    A = -np.exp(np.asarray(w[pre + "A_log"], dtype=np.float64))                    # [inner, N]
    skip = np.asarray(w[pre + "D"], dtype=np.float64)
    state = np.zeros((inner, N))
    y = np.zeros((T, inner))
    for t in range(T):
        state = np.exp(d[t][:, None] * A) * state + (d[t] * u[t])[:, None] * B[t][None, :]
        y[t] = state @ C[t] + skip * u[t]
    return linear(store(y * silu(z)), w[pre + "o"])


# ---------------------------------------------------------------------------------------------- feed-forwards
def dense_ff(w, pre: str, h, store=f32):
    inner = store(gelu_erf(linear(h, w[pre + "up"], w[pre + "up.b"])))
    return linear(inner, w[pre + "down"], w[pre + "down.b"])


def choose(scores, top: int):
    """Indices of the `top` largest scores of every row, the lowest index among equals first."""
    order = np.argsort(-scores, axis=-1, kind="stable")
    return order[:, :top]


def routed_ff(w, pre: str, m, h, store=f32):
    T = h.shape[0]
    top = m["router"]["top"]
    s = 1.0 / (1.0 + np.exp(-linear(h, w[pre + "router"])))
    chosen = choose(s, top)
    out = np.zeros((T, h.shape[1]))
    for t in range(T):
        for e in chosen[t]:
            v = store(s[t, e] * h[t])
            gate, up = linear(v, w[f"{pre}e{e}.gate"]), linear(v, w[f"{pre}e{e}.up"])
            out[t] += linear(store(silu(gate) * up), w[f"{pre}e{e}.down"])
    return out


def feed_forward(w, pre: str, m, h, store=f32):
    if m["kind"] == "dense":
        return dense_ff(w, pre, h, store)
    if m["kind"] == "moe":
        return routed_ff(w, pre, m, h, store)
    raise ValueError(m["kind"])


# ---------------------------------------------------------------------------------------------- the model
def forward(w, cfg, tokens, store=f32, rows=None, streams=None):
    """Logits [len(rows) or T, vocab] of the whole sequence.  `streams`: a list that receives x after every layer."""
    eps = float(cfg["norm"]["eps"])
    x = np.asarray(w["embed"], dtype=np.float64)[np.asarray(tokens)] * float(cfg["embedding"]["scale"])
    positions = np.arange(len(tokens))
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}."
        h = store(one_plus_norm(x, w[pre + "norm1"], eps))
        h = store(h + causal_conv(h, w[pre + "canon1"]))
        kind, m = layer["type"], layer["mixer"]
        if kind == "attention":
            x = x + attention_mixer(w, pre + "mix.", m, h, positions, eps, store)
        elif kind == "mamba2":
            x = x + mamba2_mixer(w, pre + "mix.", m, h, eps, store)
        elif kind == "mamba1":
            x = x + mamba1_mixer(w, pre + "mix.", m, h, store)
        else:
            raise ValueError(kind)
        if layer.get("mlp") is not None:
            x = x + feed_forward(w, pre + "mlp.", layer["mlp"], store(one_plus_norm(x, w[pre + "norm2"], eps)), store)
        if streams is not None:
            streams.append(x.copy())
    if rows is not None:
        x = x[np.asarray(rows)]
    x = store(one_plus_norm(x, w["final.norm"], eps))
    return linear(x, w["head"]).astype(np.float32)


def forward_logits(w, cfg, tokens, store=f32, rows=None):
    return forward(w, cfg, tokens, store=store, rows=rows)
