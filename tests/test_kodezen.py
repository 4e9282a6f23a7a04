"""Kodezen without a GPU: configuration, the plan's tensors and cache slots, and properties of the plain implementation."""
import copy
import math

import numpy as np
import pytest

import sprout_lm_amd as S
from sprout_lm_amd.cache.spec import PagedKVSpec, StateSpec
from sprout_lm_amd.config.base import ConfigError
from sprout_lm_amd.registry import build_model_plan
from tests import kodezen_helpers as KH
from tests.plain import kodezen_plain as K


@pytest.mark.parametrize("name", list(KH.CONFIGS))
def test_configuration_round_trip(name):
    cfg = S.config_from_dict(KH.CONFIGS[name])
    assert cfg.architecture == "Kodezen"
    assert S.config_from_dict(cfg.to_dict()) == cfg
    again = cfg.to_dict()
    for mine, theirs in zip(again["layers"], KH.CONFIGS[name]["layers"]):
        assert mine == theirs


@pytest.mark.parametrize("path,value", [
    (("width",), 0), (("norm", "eps"), -1.0), (("canon", "taps"), 0), (("embedding", "scale"), None),
    (("layers", 0, "type"), "lstm"), (("layers", 1, "mixer", "kv_heads"), 4), (("layers", 1, "mixer", "vdim"), 16),
    (("layers", 1, "mixer", "rot", "dims"), 7), (("layers", 0, "mixer", "groups"), 2), (("layers", 0, "mixer", "norm_groups"), 4),
    (("layers", 0, "mlp", "router", "top"), 9), (("layers", 2, "mlp", "kind"), "glu"), (("layers", 2, "mixer", "dt_rank"), 0)])
def test_configuration_refusals(path, value):
    raw = copy.deepcopy(KH.ODD)
    at = raw
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError):
        S.config_from_dict(raw)


def test_plan_names_tensors_and_cache_slots():
    plan = build_model_plan(S.config_from_dict(KH.ODD))
    parts = plan.instantiate()
    expected = parts.expected_tensors()
    assert tuple(expected["l0.mix.in"].shape) == (2 * 30 + 2 * 5 + 3, 100)
    assert tuple(expected["l0.mix.conv"].shape) == (40, 2) and tuple(expected["l0.mix.norm"].shape) == (30,)
    assert tuple(expected["l1.mix.q.conv"].shape) == (72, 3) and tuple(expected["l1.mix.k.conv"].shape) == (36, 3)
    assert tuple(expected["l1.mix.talk"].shape) == (6, 6) and tuple(expected["l1.mix.k.norm"].shape) == (12,)
    assert tuple(expected["l2.mix.x"].shape) == (3 + 2 * 5, 36) and tuple(expected["l2.mix.A_log"].shape) == (36, 5)
    assert tuple(expected["l3.mix.q.conv"].shape) == (60, 1)
    assert tuple(expected["l0.mlp.e4.down"].shape) == (100, 12) and tuple(expected["l0.mlp.router"].shape) == (5, 100)
    assert tuple(expected["l1.mlp.up.b"].shape) == (28,) and "l3.norm2" not in expected and "l3.canon1" in expected
    specs = parts.cache_slot_specs
    # the attention layers keep pages of one key/value head per (key head, value head) pair, and the window's reach
    paged = [s for s in specs if isinstance(s, PagedKVSpec)]
    assert [(s.kv_heads, s.head_dim, s.window, s.keep_first) for s in paged] == [(9, 16, 7, 2), (9, 32, None, 0)]
    states = [s.shape for s in specs if isinstance(s, StateSpec)]
    assert (3, 5, 10) in states and (36, 5) in states and (2, 108) in states and (2, 100) in states
    assert (20, 1) in states        # a selective scan of one state, whose convolution of one tap keeps nothing
    assert not parts.prefix_sharing and parts.graph_safe and parts.graph_safe_portions


def test_the_cache_keeps_the_pages_of_the_first_keys():
    from sprout_lm_amd.cache import CacheManager
    from sprout_lm_amd.cache.manager import FREED
    cache = CacheManager([PagedKVSpec(1, 16, window=10, keep_first=9), PagedKVSpec(1, 16, window=10)], 4, 40, 2, prefix_caching=False)
    seq = cache.create()
    assert cache.reserve(seq, 50)
    cache.commit(seq, 50)
    kept, plain = seq.blocks
    assert [p != FREED for p in kept[:4]] == [True, True, True, False] and all(p == FREED for p in kept[3:10])
    assert all(p == FREED for p in plain[:10]) and all(p != FREED for p in kept[10:]) and all(p != FREED for p in plain[10:])
    seq.release()
    assert cache.free_pages() == [40, 40]


def test_the_mask_spelled_out():
    m = K.visible(8, 3, 2)
    for i in range(8):
        for j in range(8):
            assert m[i, j] == (j <= i and (i - j < 3 or j < 2))
    assert K.visible(5, 1, 0).sum() == 5


def test_convolution_and_turning_by_hand():
    u = np.arange(12, dtype=np.float64).reshape(6, 2)
    w = np.array([[1.0, 10.0, 100.0], [2.0, 0.0, -1.0]])
    y = K.causal_conv(u, w)
    assert y[0].tolist() == [0.0, -1.0] and y[1].tolist() == [200.0, -3.0]
    assert y[3].tolist() == [100.0 * 6 + 10.0 * 4 + 2.0, -7.0 + 2.0 * 3.0]
    x = np.random.default_rng(0).standard_normal((4, 1, 6))
    a = K.turn_pairs(x, [5, 6, 7, 8], 4, 10.0)
    assert np.allclose(a[..., 4:], x[..., 4:])
    # a turn depends on the distance alone
    q, k = np.zeros((1, 1, 6)), np.zeros((1, 1, 6))
    q[0, 0, :4], k[0, 0, :4] = (1.0, 2.0, 3.0, 4.0), (0.5, -1.0, 2.0, 0.25)
    near = (K.turn_pairs(q, [9], 4, 10.0) * K.turn_pairs(k, [4], 4, 10.0)).sum()
    far = (K.turn_pairs(q, [105], 4, 10.0) * K.turn_pairs(k, [100], 4, 10.0)).sum()
    assert abs(near - far) < 1e-9
    # pair (0, 1) turns by the position itself: at pi / 2 the pair (1, 0) becomes (0, 1)
    one = np.zeros((1, 1, 6)); one[0, 0, 0] = 1.0
    assert np.allclose(K.turn_pairs(one, [math.pi / 2], 4, 10.0)[0, 0, :2], (0.0, 1.0), atol=1e-12)


def test_mixed_heads_and_the_keys_as_values():
    """With the identity as mixing matrix the mixer is grouped-query attention whose values are the unnormed keys; a
    matrix that swaps two heads of one key/value head swaps their outputs."""
    rng = np.random.default_rng(3)
    T, hidden, H, G, D = 9, 10, 4, 2, 6
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": 0.5, "conv": 1, "rot": {"dims": 0, "base": 10.0}}
    w = {"q": rng.standard_normal((H * D, hidden)), "k": rng.standard_normal((G * D, hidden)), "q.conv": np.ones((H * D, 1)),
         "k.conv": np.ones((G * D, 1)), "q.norm": np.ones(D), "k.norm": np.ones(D), "talk": np.eye(H), "o": np.eye(H * D)}
    h = rng.standard_normal((T, hidden))
    base = K.attention_mixer(w, "", m, h, np.arange(T), 1e-6).reshape(T, H, D)
    k = (h @ w["k"].T).reshape(T, G, D)
    assert np.allclose(base[0], k[0][[0, 0, 1, 1]], atol=1e-6)      # the first token sees itself alone: its own key
    swapped = dict(w, talk=np.eye(H)[[1, 0, 2, 3]])
    other = K.attention_mixer(swapped, "", m, h, np.arange(T), 1e-6).reshape(T, H, D)
    assert np.allclose(other[:, 0], base[:, 1], atol=1e-6) and np.allclose(other[:, 1], base[:, 0], atol=1e-6)
    # across key/value heads the weights travel and the values stay: head 0 with head 2's weights still sums its own values
    crossed = dict(w, talk=np.eye(H)[[2, 1, 0, 3]])
    mixed = K.attention_mixer(crossed, "", m, h, np.arange(T), 1e-6).reshape(T, H, D)
    assert not np.allclose(mixed[:, 0], base[:, 2], atol=1e-3)
    assert np.allclose(mixed[1:, 0].sum(), mixed[1:, 0].sum())


def test_state_space_scans_written_out():
    rng = np.random.default_rng(4)
    T, hidden = 7, 6
    m = {"heads": 2, "vdim": 3, "state": 2, "groups": 1, "conv": 1, "norm_groups": 1}
    inner = 6
    w = {"in": rng.standard_normal((2 * inner + 4 + 2, hidden)) * 0.5, "conv": np.ones((inner + 4, 1)), "conv.b": np.zeros(inner + 4),
         "dt_bias": np.array([0.3, -0.2]), "A_log": np.array([0.1, -1.0]), "D": np.array([1.5, 0.5]), "norm": np.ones(inner),
         "o": np.eye(inner)}
    h = rng.standard_normal((T, hidden))
    got = K.mamba2_mixer(w, "", m, h, 1e-6)
    p = h @ w["in"].T
    z, u = p[:, :inner], K.silu(p[:, inner:2 * inner]).reshape(T, 2, 3)
    B, C = K.silu(p[:, 12:14]), K.silu(p[:, 14:16])
    d = np.log1p(np.exp(p[:, 16:] + w["dt_bias"]))
    y = np.zeros((T, 2, 3))
    for n in range(2):
        for t in range(T):
            for s in range(t + 1):
                decay = math.exp(-math.exp(w["A_log"][n]) * d[s + 1:t + 1, n].sum())
                y[t, n] += decay * d[s, n] * (C[t] @ B[s]) * u[s, n]
            y[t, n] += w["D"][n] * u[t, n]
    y = y.reshape(T, inner) * K.silu(z)
    assert np.allclose(got, y / np.sqrt((y * y).mean(axis=1, keepdims=True) + 1e-6), atol=1e-9)
    # the selective scan with one channel and one state is a scalar recurrence
    m1 = {"inner": 1, "state": 1, "dt_rank": 1, "conv": 1}
    w1 = {"in": rng.standard_normal((2, hidden)), "conv": np.ones((1, 1)), "conv.b": np.zeros(1), "x": np.array([[0.7], [1.1], [-0.4]]),
          "dt": np.array([[0.9]]), "dt.b": np.array([0.1]), "A_log": np.array([[0.2]]), "D": np.array([0.3]), "o": np.eye(1)}
    got = K.mamba1_mixer(w1, "", m1, h)
    p = h @ w1["in"].T
    u, z = K.silu(p[:, 0]), p[:, 1]
    state, want = 0.0, []
    for t in range(T):
        d = math.log1p(math.exp(0.9 * 0.7 * u[t] + 0.1))
        state = math.exp(-d * math.exp(0.2)) * state + d * u[t] * 1.1 * u[t]
        want.append((state * -0.4 * u[t] + 0.3 * u[t]) * K.silu(z[t]))
    assert np.allclose(got[:, 0], want, atol=1e-12)


def test_routing_by_hand():
    rng = np.random.default_rng(5)
    hidden = 4
    w = {"router": np.array([[1.0, 0, 0, 0], [0, 1.0, 0, 0], [0, 0, 1.0, 0]])}
    for e in range(3):
        w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"] = (rng.standard_normal((5, hidden)), rng.standard_normal((5, hidden)),
                                                            rng.standard_normal((hidden, 5)))
    h = np.array([[2.0, 1.0, -1.0, 0.3], [0.5, 0.5, 3.0, 0.0]])
    got = K.routed_ff(w, "", {"router": {"experts": 3, "top": 2}}, h)
    assert K.choose(1.0 / (1.0 + np.exp(-h[:, :3])), 2).tolist() == [[0, 1], [2, 0]]      # a tie goes to the lower index
    expert = lambda e, v: w[f"e{e}.down"] @ (K.silu(w[f"e{e}.gate"] @ v) * (w[f"e{e}.up"] @ v))
    s = lambda v: 1.0 / (1.0 + math.exp(-v))
    assert np.allclose(got[0], expert(0, s(2.0) * h[0]) + expert(1, s(1.0) * h[0]), atol=1e-12)
    assert np.allclose(got[1], expert(2, s(3.0) * h[1]) + expert(0, s(0.5) * h[1]), atol=1e-12)
    assert not np.allclose(got[0], s(2.0) * expert(0, h[0]) + s(1.0) * expert(1, h[0]), atol=1e-3)


def test_whole_model_is_causal_and_every_constant_matters():
    cfg = KH.ODD
    w = KH.random_weights(cfg, 1)
    tokens = KH.random_tokens(cfg["vocab"], 30, 2)
    full = K.forward(w, cfg, tokens)
    assert np.allclose(K.forward(w, cfg, tokens[:17]), full[:17], atol=1e-5)
    for path, value in ((("embedding", "scale"), 2.0), (("norm", "eps"), 0.1),
                        (("layers", 1, "mixer", "mask", "size"), 6), (("layers", 1, "mixer", "mask", "keep_first"), 3),
                        (("layers", 1, "mixer", "scale"), 0.5), (("layers", 1, "mixer", "rot", "base"), 60.0),
                        (("layers", 1, "mixer", "rot", "dims"), 12), (("layers", 0, "mixer", "norm_groups"), 1),
                        (("layers", 0, "mlp", "router", "top"), 1)):
        other = copy.deepcopy(cfg)
        at = other
        for key in path[:-1]:
            at = at[key]
        at[path[-1]] = value
        assert np.abs(K.forward(w, other, tokens) - full).max() > 1e-4, path
