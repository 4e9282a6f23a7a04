"""Morarax without a GPU: the configuration's round trips and refusals, the plan's tensors and cache slots, and
properties of the plain implementation itself."""
import copy

import numpy as np
import pytest

import sprout_lm_amd as S
from sprout_lm_amd.config.base import ConfigError
from sprout_lm_amd.registry import build_model_plan
from tests import morarax_helpers as MH
from tests.plain import morarax_plain as M


@pytest.mark.parametrize("name", sorted(MH.CONFIGS))
def test_configuration_round_trip(name):
    raw = MH.CONFIGS[name]
    cfg = S.config_from_dict(raw)
    assert cfg.architecture == "Morarax" and cfg.to_dict() == raw
    assert S.config_from_dict(cfg.to_dict()) == cfg
    assert cfg.vocab_size == raw["vocab"] and cfg.hidden_size == raw["width"]


def broken(path, value, base="general"):
    raw = copy.deepcopy(MH.CONFIGS[base])
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is KeyError:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return raw


@pytest.mark.parametrize("path,value", [
    (("vocab",), 0), (("width",), "wide"), (("norm",), None), (("layers",), []), (("residual_mult",), KeyError),
    (("logit_scale",), -1.0), (("layers", 0, "type"), "attention_2"), (("layers", 0, "mixer", "heads"), 3),
    (("layers", 0, "mixer", "rot"), KeyError), (("layers", 0, "mixer", "rot", "dims"), 7), (("layers", 0, "mixer", "rot", "dims"), 40),
    (("layers", 0, "mixer", "scale"), 0), (("layers", 0, "mlp", "kind"), "moe"), (("layers", 1, "mixer", "blocks"), 5),
    (("layers", 1, "mixer", "conv"), 0), (("layers", 2, "mixer", "decay"), [0.9]), (("layers", 2, "mixer", "decay"), [0.9, 1.5]),
    (("layers", 3, "mixer", "rot", "scaling", "factor"), KeyError), (("layers", 2, "mixer", "vdim"), KeyError),
])
def test_configuration_refusals(path, value):
    with pytest.raises(ConfigError):
        S.config_from_dict(broken(path, value))


def test_plan_names_every_tensor_and_cache_slot():
    from sprout_lm_amd.cache.spec import PagedKVSpec, StateSpec
    plan = build_model_plan(S.config_from_dict(MH.ODD))
    parts = plan.instantiate()
    names = parts.expected_tensors()
    assert {"embed", "final.norm", "head", "l0.norm1", "l0.ls1", "l0.ls2", "l2.ls1", "l0.mix.g", "l1.mix.g", "l2.mix.ra.b",
            "l2.mix.conv.b", "l2.mix.lam", "l4.mix.y.b", "l5.mix.q", "l1.mlp.down"} <= set(names)
    assert "l2.ls2" not in names and "l2.mlp.gate" not in names and "l0.norm2" not in names       # no feed-forward there
    assert names["l1.mix.g"].shape == (6, 100) and names["l0.mix.g"].shape == (18, 100)
    assert names["l2.mix.ra"].shape == (3, 20, 20) and names["l2.mix.conv"].shape == (60, 4)
    assert names["l4.mix.conv"].shape == (36, 1)
    # retention: one state; attention: pages at the common width of keys and values; recurrence: the state and, with more
    # than one tap, the convolution's inputs
    assert parts.cache_slot_specs == [
        StateSpec((3, 20, 6)), PagedKVSpec(2, 16), StateSpec((60,)), StateSpec((3, 60)), PagedKVSpec(3, 32), StateSpec((36,)),
        StateSpec((2, 10, 30))]
    assert not parts.prefix_sharing and parts.graph_safe and parts.graph_safe_portions
    only_attention = build_model_plan(S.config_from_dict(MH.ATTENTION)).instantiate()
    assert only_attention.prefix_sharing          # pages alone: a function of the tokens before them


def test_blended_frequencies():
    """Without scaling: base^(-2i/dims) and magnitude 1.  With it: fast pairs keep their frequency, slow ones are divided
    by the factor, those in between are blended; the magnitude is 0.1 ln(factor) + 1."""
    freq, magnitude = M.pair_frequencies(MH.rot(8, 100.0))
    assert np.allclose(freq, 100.0 ** (-np.arange(4) / 4.0)) and magnitude == 1.0
    rotation = MH.rot(32, 10000.0, (4.0, 512, 32.0, 1.0))
    freq, magnitude = M.pair_frequencies(rotation)
    plain = 10000.0 ** (-np.arange(16) / 16.0)
    assert abs(magnitude - (0.1 * np.log(4.0) + 1.0)) < 1e-15
    assert np.allclose(freq[:2], plain[:2]) and np.allclose(freq[-2:], plain[-2:] / 4.0)
    ratio = freq / plain
    assert np.all(np.diff(ratio) <= 1e-12) and ratio[0] == 1.0 and abs(ratio[-1] - 0.25) < 1e-12
    # the engine's table is the same function
    from sprout_lm_amd.parts import make_part
    part = make_part("position", "rotary_neox", head_dim=32, theta=10000.0, rotary_dim=32, scaling=rotation["scaling"])
    assert np.allclose(part.frequencies().numpy(), freq, rtol=1e-14) and part.magnitude == magnitude


def test_turning_depends_on_distance_alone_and_leaves_the_rest():
    rng = np.random.default_rng(0)
    rotation = MH.rot(8, 50.0)
    q, k = rng.normal(size=(1, 1, 12)), rng.normal(size=(1, 1, 12))
    dots = [float((M.turn_halves(q, [p + 5], rotation) * M.turn_halves(k, [p], rotation)).sum()) for p in (0, 3, 1000)]
    assert np.allclose(dots, dots[0])
    assert np.array_equal(M.turn_halves(q, [77], rotation)[..., 8:], q[..., 8:])
    assert np.allclose(M.turn_halves(q, [0], rotation), q)


def test_the_extra_one_in_the_denominator():
    """One key of score s gets exp(s) / (1 + exp(s)); weights never sum to 1; very negative scores leave next to nothing."""
    allowed = np.ones((1, 1), bool)
    assert np.allclose(M.softmax_plus_one(np.array([[0.0]]), allowed), 0.5)
    assert np.allclose(M.softmax_plus_one(np.array([[2.0]]), allowed), np.exp(2.0) / (1 + np.exp(2.0)))
    w = M.softmax_plus_one(np.array([[1.0, 2.0, 3.0]]), np.array([[True, True, False]]))
    assert w[0, 2] == 0.0 and np.allclose(w[0, :2], np.exp([1.0, 2.0]) / (1 + np.exp(1.0) + np.exp(2.0)))
    assert M.softmax_plus_one(np.full((1, 4), -40.0), np.ones((1, 4), bool)).sum() < 1e-15
    assert np.allclose(M.softmax_plus_one(np.full((1, 4), 800.0), np.ones((1, 4), bool)), 0.25)      # no overflow


def test_convolution_and_recurrence_written_out():
    x = np.arange(1.0, 9.0).reshape(4, 2)
    kw = np.array([[1.0, 10.0, 100.0], [0.0, 0.0, 2.0]])
    out = M.causal_conv(x, kw, [0.5, 0.0])
    assert np.allclose(out[:, 0], [100.5, 300 + 10 + 0.5, 500 + 30 + 1 + 0.5, 700 + 50 + 3 + 0.5])
    assert np.allclose(out[:, 1], 2 * x[:, 1])
    u = np.array([[1.0], [2.0], [3.0]])
    r, i, lam = np.full((3, 1), 0.5), np.full((3, 1), 0.25), np.array([0.3])
    a = np.exp(-8 * 0.5 * np.log1p(np.exp(0.3)))
    b = np.sqrt(1 - a * a) * 0.25
    states = M.gated_linear_recurrence(u, r, i, lam)
    assert np.allclose(states[:, 0], [b * 1, a * b * 1 + b * 2, a * (a * b + 2 * b) + 3 * b])
    gates = M.block_gate(np.array([[1.0, 2.0, 3.0, 4.0]]), np.array([[[1.0, 0.0], [0.0, -1.0]], [[0.5, 0.5], [0.0, 0.0]]]),
                         np.array([[0.0, 1.0], [0.0, 0.0]]))
    assert np.allclose(gates, M.sigmoid(np.array([[1.0, -1.0, 3.5, 0.0]])))


def test_retention_is_a_decayed_sum_without_a_denominator():
    """o_t = sum over j <= t of decay^(t - j) (q_t . k_j dim^(-1/2)) v_j, then the head's unit norm and gate."""
    rng = np.random.default_rng(2)
    T, D, V, hidden = 6, 4, 3, 5
    w = {"q": rng.normal(size=(D, hidden)), "k": rng.normal(size=(D, hidden)), "v": rng.normal(size=(V, hidden)),
         "g": rng.normal(size=(V, hidden)), "o": np.eye(V)}
    h = rng.normal(size=(T, hidden))
    m = {"heads": 1, "dim": D, "vdim": V, "decay": [0.8], "rot": MH.rot(0)}
    got = M.retention_mixer(w, "", m, h, np.arange(T), 1e-6, store=lambda x: np.asarray(x, np.float64))
    q, k, v = h @ w["q"].T, h @ w["k"].T * D ** -0.5, h @ w["v"].T
    o = np.stack([sum(0.8 ** (t - j) * (q[t] @ k[j]) * v[j] for j in range(t + 1)) for t in range(T)])
    want = o / np.sqrt((o * o).mean(-1, keepdims=True) + 1e-6) * M.silu(h @ w["g"].T)
    assert np.allclose(got, want)


def test_whole_model_is_causal_and_uses_every_constant():
    cfg = copy.deepcopy(MH.STATES)
    w = MH.random_weights(cfg, 1)
    tokens = MH.random_tokens(cfg["vocab"], 12, 0)
    base = M.forward(w, cfg, tokens)
    other = M.forward(w, cfg, tokens[:8] + [t ^ 1 for t in tokens[8:]])
    assert np.array_equal(base[:8], other[:8]) and not np.allclose(base[8:], other[8:])
    for key, value in (("residual_mult", 0.9), ("logit_scale", 3.0)):
        changed = dict(cfg, **{key: value})
        assert not np.allclose(M.forward(w, changed, tokens), base)
    doubled = M.forward(w, dict(cfg, logit_scale=2 * cfg["logit_scale"]), tokens)
    assert np.allclose(doubled, 2 * base, rtol=1e-6)
