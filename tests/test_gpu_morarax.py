"""Morarax on the GPU: every mechanism alone against its plain function, then whole models cut into steps in
different ways, then generation through the engine's entry point and scheduler."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import morarax_helpers as MH
from tests import traces
from tests.plain import morarax_plain as M
from tests.test_gpu_megozen import Harness, dev

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]


def rounded(x, dtype):
    return M.bf16_round(x) if dtype == torch.bfloat16 else np.asarray(x, np.float32)


def store_of(dtype):
    return M.bf16_round if dtype == torch.bfloat16 else M.f32


def close(got, want, dtype, what, f32=2e-5, bf16=2e-2):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    bound = (f32 if dtype == torch.float32 else bf16) * max(1.0, float(np.abs(want).max()))
    err = float(np.abs(got - want).max())
    assert err <= bound, f"{what}: off by {err:.3e} (bound {bound:.1e})"


def weights_for(part, rng, dtype, scales=None):
    """Random tensors for a part, by the last piece of their local names."""
    scales = scales or {}
    out = {}
    for name, spec in part.tensors().items():
        last = name.split(".")[-1]
        if last == "b":
            a = rng.normal(0, 0.2, spec.shape)
        elif last == "conv":
            a = rng.normal(0, 0.5, spec.shape)
        elif last == "lam":
            a = rng.normal(-1, 1, spec.shape)
        elif last in ("ra", "ri"):
            a = rng.normal(0, 0.3, spec.shape)
        else:
            a = rng.normal(0, scales.get(last, 0.15), spec.shape)
        out[name] = rounded(a, dtype).reshape(spec.shape)
    return out


def run_in_portions(part, specs, dtype, inputs, steps, hidden, page=8):
    """Feed the sequences `inputs` (rows of the mixer's input each) through `part` in the portions `steps` (one tuple of
    token counts per step, a count per sequence) beside each other; returns what the part added, per sequence."""
    harness = Harness(specs, dtype, page=page, pages=96, slots=len(inputs))
    seqs = [harness.cache.create() for _ in inputs]
    fed = [0] * len(inputs)
    got = [np.zeros((len(x), hidden), np.float32) for x in inputs]
    for step in steps:
        batch = [(i, min(n, len(inputs[i]) - fed[i])) for i, n in enumerate(step) if n and fed[i] < len(inputs[i])]
        if not batch:
            continue
        ctx, entries = harness.context([(seqs[i], [0] * n) for i, n in batch])
        h = torch.cat([dev(inputs[i][fed[i]:fed[i] + n], dtype) for i, n in batch])
        residual = torch.zeros(h.shape[0], hidden, device=DEV)
        keys = list(part.cache_spec()) if isinstance(part.cache_spec(), dict) else None
        cache = {k: harness.view(ctx, j) for j, k in enumerate(keys)} if keys else harness.view(ctx, 0)
        part.forward(ctx, h, residual, cache)
        out = residual.cpu().numpy()
        harness.commit(entries)
        row = 0
        for i, n in batch:
            got[i][fed[i]:fed[i] + n] = out[row:row + n]
            fed[i] += n
            row += n
    assert fed == [len(x) for x in inputs]
    return got


def specs_of(part):
    spec = part.cache_spec()
    return list(spec.values()) if isinstance(spec, dict) else [spec]


PORTIONS = [(16, 1), (5, 9), (1, 1), (2, 3), (13, 8), (1, 2), (40, 40), (1, 1), (1, 1), (250, 250)]


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_rotation_table_with_blended_frequencies(dtype):
    """Cosines and sines of the half-split rotation at positions up to a million, plain and with blended frequencies
    and their magnitude."""
    from sprout_lm_amd.engine.batch import StepContext, Workspace
    from sprout_lm_amd.parts import make_part
    for rotation in (MH.rot(24, 300.0), MH.rot(16, 100.0, (2.0, 32, 4.0, 1.0)), MH.rot(40, 1e6, (8.0, 64, 16.0, 1.0))):
        part = make_part("position", "rotary_neox", head_dim=48, theta=rotation["base"], rotary_dim=rotation["dims"],
                         scaling=rotation.get("scaling"))
        part.prepare(DEV, dtype)
        freq, magnitude = M.pair_frequencies(rotation)
        assert np.allclose(part.frequencies().numpy(), freq, rtol=1e-14) and abs(part.magnitude - magnitude) < 1e-15
        positions = np.array([0, 1, 2, 77, 4095, 1000003], dtype=np.int32)
        ctx = StepContext(Workspace(DEV), dtype, 0)
        ctx.positions, ctx.n_tokens = torch.from_numpy(positions).to(DEV), len(positions)
        table = part.table(ctx).cpu().numpy()
        angle = positions[:, None].astype(np.float64) * freq[None, :]
        # float32 angles at a position of a million are off by that position times 6e-8
        bound = 2e-6 if dtype == torch.float32 else 1e-7 * 1000003 * float(freq.max()) + 2e-6
        assert np.abs(table[..., 0] - np.cos(angle) * magnitude).max() <= bound
        assert np.abs(table[..., 1] - np.sin(angle) * magnitude).max() <= bound


@pytest.mark.parametrize("dtype", DTYPES)
def test_scaled_sum_head_gate_and_logit_scale(dtype):
    from sprout_lm_amd import ops
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(3)
    T, H = 37, 100
    x, a, b = (rng.normal(0, 1, (T, H)).astype(np.float32) for _ in range(3))
    sa, sb = rounded(1 + rng.normal(0, 0.3, H), dtype), rounded(rng.normal(0, 1, H), dtype)
    one = make_part("scale", "layer_scale", size=H, multiplier=0.7, tensor="ls1")
    two = make_part("scale", "layer_scale", size=H, multiplier=0.7, tensor="ls2")
    assert list(one.tensors()) == ["ls1"]
    one.bind({"ls1": dev(sa, dtype)}); two.bind({"ls2": dev(sb, dtype)})
    residual = dev(x)
    one.add(None, residual, dev(a), two, dev(b))
    close(residual.cpu().numpy(), x + 0.7 * (sa * a.astype(np.float64) + sb * b), torch.float32, "two branches", f32=1e-6)
    residual = dev(x)
    one.add(None, residual, dev(a))
    close(residual.cpu().numpy(), x + 0.7 * sa * a.astype(np.float64), torch.float32, "one branch", f32=1e-6)
    heads, width = 5, 12
    rows = rounded(rng.normal(0, 1, (T, heads * width)), dtype)
    gates = rounded(rng.normal(0, 2, (T, 9)), dtype)
    t = dev(rows, dtype)
    ops.head_gate(t, dev(gates, dtype), 3, heads, width)
    want = rows.reshape(T, heads, width) * M.sigmoid(gates[:, 3:3 + heads])[:, :, None]
    close(t.float().cpu().numpy(), want.reshape(T, -1), dtype, "head gate", bf16=1e-2)
    head = make_part("head", "linear_head", vocab=41, hidden=H, tied=False, tensor="head", scale=0.3)
    table = rounded(rng.normal(0, 0.2, (41, H)), dtype)
    head.bind({"head": dev(table, dtype)})
    h = rounded(rng.normal(0, 1, (4, H)), dtype)
    logits = torch.empty(4, 41, device=DEV)
    head.forward(None, dev(h, dtype), logits)
    close(logits.cpu().numpy(), M.linear(h, table) * 0.3, torch.float32, "scaled logits", f32=1e-5)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,inner,T", [(100, 28, 7), (128, 96, 5), (128, 96, 70), (64, 64, 300)])
def test_relu_gated_feed_forward(dtype, hidden, inner, T):
    """down(max(gate, 0) * up) on every path a gated product takes: few tokens, many, sizes in no whole eights."""
    from sprout_lm_amd.engine.batch import StepContext, Workspace
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(hidden + T)
    part = make_part("feed_forward", "gated_mlp", hidden=hidden, inner=inner, activation="relu", tensors=("gate", "up", "down"))
    w = weights_for(part, rng, dtype)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    x = rounded(rng.normal(0, 1, (T, hidden)), dtype)
    residual = torch.zeros(T, hidden, device=DEV)
    part.forward(StepContext(Workspace(DEV), dtype, 0), dev(x, dtype), residual)
    close(residual.cpu().numpy(), M.dense_ff(w, "", x, store_of(dtype)), dtype, "relu feed-forward")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width,blocks,taps", [(60, 3, 4), (36, 1, 1), (192, 2, 3), (128, 8, 2), (640, 1, 5)])
def test_gated_recurrence_alone_in_portions(dtype, width, blocks, taps):
    """Two sequences in uneven portions beside each other (portions shorter than the convolution among them), then a long
    portion: the state and the convolution's last inputs go from step to step."""
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(width + taps)
    hidden = 72
    part = make_part("mixer", "gated_linear_recurrence", hidden=hidden, width=width, blocks=blocks, taps=taps)
    w = weights_for(part, rng, dtype)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    inputs = [rounded(rng.normal(0, 1, (n, hidden)), dtype) for n in (281, 266)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    for x, out in zip(inputs, got):
        want = M.rglru_mixer(w, "", {"width": width, "blocks": blocks, "conv": taps}, x, store_of(dtype))
        close(out, want, dtype, f"recurrence of {width} channels")


def test_recurrence_keeps_a_far_token():
    """A channel whose decay is almost 1 still holds, 600 tokens later, what a single early token put there; a channel
    whose decay is small has lost it.  lam decides: softplus(lam) tiny or large."""
    from sprout_lm_amd.parts import make_part
    dtype, hidden, width = torch.float32, 16, 16
    part = make_part("mixer", "gated_linear_recurrence", hidden=hidden, width=width, blocks=1, taps=1)
    rng = np.random.default_rng(0)
    w = weights_for(part, rng, dtype)
    w["lam"] = np.where(np.arange(width) % 2 == 0, -12.0, 3.0).astype(np.float32)     # even channels remember
    w["conv"] = np.ones((width, 1), np.float32)
    w["x"] = np.eye(width, hidden, dtype=np.float32)
    for name in ("ra", "ri", "ra.b", "ri.b", "x.b", "conv.b"):      # both gates at one half, the channels' input the mixer's own
        w[name] = np.zeros_like(w[name])
    w["y.b"] = np.ones(width, np.float32)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    x = np.zeros((640, hidden), np.float32)
    x[3] = 50.0                                                                          # the one token that matters
    x[4:] = rng.normal(0, 0.01, (636, hidden))
    got = run_in_portions(part, specs_of(part), dtype, [x], [(5,), (300,), (1,), (1,), (333,)], hidden)[0]
    m = {"width": width, "blocks": 1, "conv": 1}
    want = M.rglru_mixer(w, "", m, x)
    close(got, want, dtype, "far token")
    # the premise of the test: without that token the last output is another one, and only through the channels that remember
    without = np.concatenate([x[:3], 0 * x[3:4], x[4:]])
    moved = np.abs(want[-1] - M.rglru_mixer(w, "", m, without)[-1]).max()
    forgetful = dict(w, lam=np.full(width, 3.0, np.float32))
    lost = np.abs(M.rglru_mixer(forgetful, "", m, x)[-1] - M.rglru_mixer(forgetful, "", m, without)[-1]).max()
    assert moved > 0.2 * np.abs(want[-1]).max() and lost < 1e-6 * moved


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,vdim,dims", [(3, 20, 6, 8), (2, 32, 64, 32), (4, 64, 16, 16), (2, 10, 30, 0), (1, 128, 128, 64),
                                                  (2, 256, 64, 32), (2, 48, 200, 48), (1, 130, 256, 64), (2, 24, 300, 0)])
def test_retention_alone_in_portions(dtype, heads, dim, vdim, dims):
    from sprout_lm_amd.models.plan import PartPlan
    rng = np.random.default_rng(dim + vdim)
    hidden, eps = 48, 1e-4
    decay = [1.0, 0.5, 0.97, 0.999][:heads]
    rotation = MH.rot(dims, 700.0)
    position = PartPlan("position", "rotary_neox", {"head_dim": dim, "theta": 700.0, "rotary_dim": dims}) if dims else \
        PartPlan("position", "none", {"head_dim": dim})
    part = PartPlan("mixer", "retention", {"hidden": hidden, "heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                                           "eps": eps, "position": position}).make()
    w = weights_for(part, rng, dtype)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    part.prepare(DEV, dtype)
    inputs = [rounded(rng.normal(0, 1, (n, hidden)), dtype) for n in (281, 266)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay, "rot": rotation}
    for x, out in zip(inputs, got):
        want = M.retention_mixer(w, "", m, x, np.arange(len(x)), eps, store_of(dtype))
        close(out, want, dtype, f"retention with heads of {dim} and {vdim}")


def test_retention_reads_a_far_key():
    """With q = k = the input itself, a query equal to one early key and a value there far from all others: the head whose
    decay is 1 returns that value from 500 tokens back, past portions and single tokens; the head whose decay is 0.9 has
    forgotten it."""
    from sprout_lm_amd.models.plan import PartPlan
    dtype, heads, dim, vdim = torch.float32, 2, 16, 16
    hidden = heads * dim + 8          # the last 8 numbers of the input reach the values alone
    part = PartPlan("mixer", "retention", {"hidden": hidden, "heads": heads, "dim": dim, "vdim": vdim, "decay": [1.0, 0.9],
                                           "eps": 1e-6, "position": PartPlan("position", "none", {"head_dim": dim})}).make()
    rng = np.random.default_rng(1)
    w = weights_for(part, rng, dtype)
    w["q"] = w["k"] = np.eye(heads * dim, hidden, dtype=np.float32)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    part.prepare(DEV, dtype)
    x = rng.normal(0, 0.02, (520, hidden)).astype(np.float32)
    x[7] = 0.0
    x[7, 0] = x[7, dim] = 30.0           # the key that stands out, in both heads
    x[7, -8:] = 9.0                       # with a value of its own
    x[-1, :heads * dim] = x[7, :heads * dim]     # and the query that asks for it
    got = run_in_portions(part, specs_of(part), dtype, [x], [(9,), (250,), (2,), (1,), (258,)], hidden)[0]
    m = {"heads": heads, "dim": dim, "vdim": vdim, "decay": [1.0, 0.9], "rot": MH.rot(0)}
    want = M.retention_mixer(w, "", m, x, np.arange(len(x)), 1e-6)
    close(got, want, dtype, "far key")
    # the premise of the test: without that key the last output is another one
    forgotten = M.retention_mixer(w, "", m, np.concatenate([x[:7], 0 * x[7:8], x[8:]]), np.arange(len(x)), 1e-6)
    assert np.abs(want[-1] - forgotten[-1]).max() > 0.05 * np.abs(want[-1]).max()


def attention_part(hidden, heads, kv_heads, dim, vdim, scale, rotation, eps):
    from sprout_lm_amd.models.plan import PartPlan
    position = PartPlan("position", "rotary_neox", {"head_dim": dim, "theta": rotation["base"], "rotary_dim": rotation["dims"],
                                                    "scaling": rotation.get("scaling")}) if rotation["dims"] else \
        PartPlan("position", "none", {"head_dim": dim})
    return PartPlan("mixer", "sink_attention", {"hidden": hidden, "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                                "scale": scale, "position": position, "eps": eps, "sinks": False,
                                                "sink_value": 0.0, "head_norm": True, "head_gate": True}).make()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,rotation", [
    (6, 2, 12, 10, MH.rot(12, 50.0, (4.0, 16, 8.0, 2.0))), (3, 3, 20, 24, MH.rot(0)), (4, 2, 32, 64, MH.rot(16)),
    (16, 1, 64, 32, MH.rot(32, 250.0, (8.0, 64, 16.0, 1.0))), (2, 1, 48, 80, MH.rot(24))])
def test_attention_alone_in_portions(dtype, heads, kv_heads, dim, vdim, rotation):
    """Heads normed after turning, one more 1 in the denominator, a gate per head: prompts in portions beside each
    other, then token by token over pages."""
    rng = np.random.default_rng(heads * dim)
    hidden, eps, scale = 56, 1e-5, 0.3
    part = attention_part(hidden, heads, kv_heads, dim, vdim, scale, rotation, eps)
    w = weights_for(part, rng, dtype, {"g": 0.4})
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    part.prepare(DEV, dtype)
    inputs = [rounded(rng.normal(0, 1, (n, hidden)), dtype) for n in (281, 266)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": rotation}
    for x, out in zip(inputs, got):
        want = M.attention_mixer(w, "", m, x, np.arange(len(x)), eps, store_of(dtype))
        close(out, want, dtype, f"attention with heads of {dim} and {vdim}", bf16=3e-2)


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_keys_and_the_extra_one(dtype):
    """With q = k = the input itself (unit heads after the norm): a query that equals one key among 600 scores dim * scale
    there and about 0 elsewhere, so that key's value dominates, wherever it lies (first position, a page's last and first
    place, far back) and whether the query comes in a portion or alone; and where no key matches, the 1 in the
    denominator outweighs the keys and the output all but vanishes."""
    heads, dim, vdim, scale, eps = 2, 32, 32, 0.8, 1e-6
    hidden = heads * dim + 8          # the last 8 numbers of the input reach the values alone
    part = attention_part(hidden, heads, heads, dim, vdim, scale, MH.rot(0), eps)
    rng = np.random.default_rng(5)
    w = weights_for(part, rng, dtype)
    w["q"] = w["k"] = np.eye(heads * dim, hidden, dtype=np.float32)
    w["g"] = np.zeros((heads, hidden), np.float32)
    part.bind({n: dev(a, dtype) for n, a in w.items()})
    part.prepare(DEV, dtype)
    n = 600
    # keys: sign patterns with few agreements between them (Hadamard rows would agree in none; random signs in dim / 2 +- a few)
    signs = np.where(rng.random((n, hidden)) < 0.5, -1.0, 1.0).astype(np.float32)
    flagged = [0, 7, 8, 15, 16, 300]
    x = signs.copy()
    queries = {n - 40 + i: key for i, key in enumerate(flagged)}      # in the last portion
    queries.update({n - 6 + i: key for i, key in enumerate(flagged)})  # fed one by one
    for at, key in queries.items():
        x[at, :heads * dim] = x[key, :heads * dim]
    got = run_in_portions(part, specs_of(part), dtype, [x], [(500,), (70,), (24,)] + [(1,)] * 6, hidden, page=8)[0]
    m = {"heads": heads, "kv_heads": heads, "dim": dim, "vdim": vdim, "scale": scale, "rot": MH.rot(0)}
    want = M.attention_mixer(w, "", m, x, np.arange(n), eps, store_of(dtype))
    close(got, want, dtype, "crafted keys", bf16=3e-2)
    # the premise: leaving the flagged key out changes the output by much
    for at, key in list(queries.items())[:3]:
        other = x.copy()
        other[key, :heads * dim] = -other[key, :heads * dim]
        moved = M.attention_mixer(w, "", m, other[:at + 1], np.arange(at + 1), eps)[at]
        assert np.abs(moved - want[at]).max() > 0.1 * np.abs(want[at]).max()


# ---------------------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("morarax"))
    return {name: MH.make_folder(root, name) for name in MH.CONFIGS}


def requests_for(name, lengths, seed=100):
    vocab = MH.CONFIGS[name]["vocab"]
    return {f"r{i}": MH.random_tokens(vocab, n, seed + i) for i, n in enumerate(lengths)}


def replay(folder, name, dtype, trace, max_tokens, page=None, slots=4, reused=None):
    """The engine's trace session on a pool of `max_tokens`; per step the logits rows."""
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.trace import TraceSession
    page = page or MH.PAGE[name]
    runner = ModelRunner.from_folder(folder, dtype, block_size=page, num_blocks=-(-max_tokens // page), max_sequences=slots,
                                     prefix_caching=False)
    session = TraceSession(runner)
    out, owners, holders = [], {}, {}
    for record in trace.steps:
        logits = session.run_step(record)
        out.append(None if logits is None or not logits.shape[0] else logits.cpu().numpy().copy())
        for rid, seq in session.live.items():
            if rid not in holders.setdefault(seq.state_slot, []):
                holders[seq.state_slot].append(rid)
            for g, blocks in enumerate(seq.blocks):
                for page_id in blocks:
                    if page_id >= 0 and rid not in owners.setdefault((g, page_id), []):
                        owners[(g, page_id)].append(rid)
    if reused is not None:
        reused["pages"] = sum(len(r) > 1 for r in owners.values())
        reused["slots"] = sum(len(r) > 1 for r in holders.values())
    assert all(free == total for free, total in zip(runner.cache.free_pages(), [g.pool.num_pages for g in runner.cache.groups]))
    assert not session.live
    return out


def check(folder, dtype, requests, trace, results):
    worst = 0.0
    for step, (rows, got) in enumerate(zip(trace.expected, results)):
        if not rows:
            assert got is None
            continue
        assert got.shape[0] == len(rows)
        for i, (rid, pos) in enumerate(rows):
            want = MH.plain_logits(folder, dtype, requests[rid])[pos]
            err = float(np.abs(got[i] - want).max())
            worst = max(worst, err)
            bound = MH.tolerance(dtype, want)
            if dtype == "bfloat16":     # how far bfloat16 rounding moves this row on the plain side itself (a head's unit
                # norm over a first token's near-zero score can turn a rounding into a sign)
                bound += float(np.abs(want - MH.plain_logits(folder, "float32", requests[rid])[pos]).max())
            assert err <= bound, f"step {step} request {rid} position {pos}: error {err:.3e}"
    return worst


LENGTHS = {"odd": [1, 2, 21, 70, 45, 97], "general": [1, 9, 40, 97, 150, 33, 2, 75], "states": [9, 40, 97, 33, 130, 3],
           "attention": [2, 70, 97, 33, 64, 120]}
CASES = [(n, "float32") for n in MH.CONFIGS] + [(n, "bfloat16") for n in MH.CONFIGS]


@pytest.mark.parametrize("name,dtype", CASES)
@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_replay_family(folders, name, dtype, family):
    """Whole prompts; a prompt and its last 48 tokens one by one; portions down to two tokens; four live requests in a
    pool and on state slots that hold no more, so that pages and slots are used again."""
    requests = requests_for(name, LENGTHS[name])
    roomy = 4 * 64 * (1 + max(LENGTHS[name]) // 64)
    if family == "whole":
        trace, pool = traces.whole(requests), roomy
    elif family == "tail":
        trace, pool = traces.tail_decoded(requests, tail=48), roomy
    elif family == "portions":
        trace, pool = traces.portions(requests), roomy
    else:
        trace = traces.mixed(requests, seed=7)
        pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    reused = {}
    results = replay(folders[name], name, dtype, trace, pool, reused=reused)
    if family == "mixed":
        assert reused["slots"] >= 1, f"no state slot was used again: {reused}"
        if name != "states":
            assert reused["pages"] >= 2, f"no page was used again: {reused}"
    worst = check(folders[name], dtype, requests, trace, results)
    print(f"{family} {name} {dtype}: {len(trace.steps)} steps, worst error {worst:.3e}")


@pytest.mark.parametrize("name,page,dtype", [("general", 12, "float32"), ("odd", 4, "float32"), ("attention", 64, "float32"),
                                             ("general", 24, "bfloat16")])
def test_replay_with_other_page_sizes(folders, name, page, dtype):
    requests = requests_for(name, LENGTHS[name], seed=300)
    trace = traces.mixed(requests, seed=11)
    pool = sum(sorted(-(-len(t) // 192) * 192 for t in requests.values())[-4:])
    results = replay(folders[name], name, dtype, trace, pool, page=page)
    check(folders[name], dtype, requests, trace, results)


@pytest.mark.parametrize("name,dtype", [("general", "float32"), ("states", "float32"), ("odd", "bfloat16")])
def test_long_prompts_in_long_portions(folders, name, dtype):
    """Prompts of many chunks of the recurrent mixers' long-portion kernels: whole, in long uneven portions (chunk edges
    fall anywhere), and two requests' long portions beside each other and beside single tokens."""
    requests = requests_for(name, [700, 333], seed=500)
    cut = traces.portions(requests, sizes=(200, 129, 65, 2, 64, 190, 1, 70))
    both = traces.Trace()
    a, b = requests["r0"], requests["r1"]
    both.add([("r0", 0, a[:400], range(390, 400)), ("r1", 0, b[:150], [149])])
    both.add([("r0", 400, a[400:401], [0]), ("r1", 150, b[150:], range(0, 183, 7))], end=["r1"])
    both.add([("r0", 401, a[401:], range(0, 299, 5))], end=["r0"])
    for trace in (traces.whole(requests), cut, both):
        results = replay(folders[name], name, dtype, trace, 1280)
        check(folders[name], dtype, requests, trace, results)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other(folders, dtype):
    """Whole, token-by-token and portioned replays give the same logits beyond rounding."""
    name = "general"
    requests = requests_for(name, [90])
    rows_of = {}
    for family, trace in (("whole", traces.whole(requests)), ("tail", traces.tail_decoded(requests, tail=89)),
                          ("portions", traces.portions(requests))):
        results = replay(folders[name], name, dtype, trace, 256)
        rows_of[family] = {key: got[i] for expect, got in zip(trace.expected, results) for i, key in enumerate(expect)}
    bound = 1e-5 if dtype == "float32" else 3e-2
    for key, row in rows_of["whole"].items():
        for other in ("tail", "portions"):
            if key in rows_of[other]:
                assert np.abs(row - rows_of[other][key]).max() <= bound * max(1.0, np.abs(row).max()), (key, other)


def test_first_tokens_and_long_decoding(folders):
    """Positions 0, 1, 2, ... fed one by one from the very first token, 260 in a row."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    for name, dtype in (("general", "float32"), ("odd", "float32"), ("states", "bfloat16")):
        tokens = MH.random_tokens(MH.CONFIGS[name]["vocab"], 260, 9)
        runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=40, max_sequences=2,
                                         prefix_caching=False)
        seq = runner.cache.create()
        want = MH.plain_logits(folders[name], dtype, tokens)
        for p, token in enumerate(tokens):
            assert runner.cache.reserve(seq, p + 1)
            got = runner.step([StepEntry(seq, [token], [0])]).cpu().numpy()[0]
            assert np.abs(got - want[p]).max() <= MH.tolerance(dtype, want[p]), f"{name} {dtype} position {p}"
        seq.release()


def test_a_state_slot_starts_from_zero_again(folders):
    """A request that takes over the slot of a finished one computes what it computes on a fresh engine."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    name, dtype = "states", "float32"
    runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=16, max_sequences=1, prefix_caching=False)
    vocab = MH.CONFIGS[name]["vocab"]
    for seed in (1, 2, 3):
        tokens = MH.random_tokens(vocab, 50, seed)
        seq = runner.cache.create()
        assert seq.state_slot == 0 and runner.cache.reserve(seq, 50)
        got = runner.step([StepEntry(seq, tokens, [49])]).cpu().numpy()[0]
        want = MH.plain_logits(folders[name], dtype, tokens)[49]
        assert np.abs(got - want).max() <= MH.tolerance(dtype, want)
        seq.release()


def test_trace_replay_program(folders, tmp_path):
    """The replay program as a user runs it, on a model it picks by the folder's config.json."""
    name, dtype = "general", "float32"
    requests = requests_for(name, [33, 70, 20, 64, 45])
    trace = traces.mixed(requests, seed=3)
    pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    out = tmp_path / "logits"
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name],
                             "--dtype", dtype, "--out", str(out), "--max-tokens", str(pool)],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for record in trace.steps:
            proc.stdin.write(json.dumps(record) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {record['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = MH.CONFIGS[name]["vocab"]
    results = [np.fromfile(out / f"{r['step']}.f32", dtype="<f4").reshape(len(rows), vocab) if rows else None
               for r, rows in zip(trace.steps, trace.expected)]
    check(folders[name], dtype, requests, trace, results)


# ---------------------------------------------------------------------------------------------- generation
def plain_greedy(folder, dtype, prompt, steps):
    history, out = list(prompt), []
    for _ in range(steps):
        token = int(np.argmax(MH.plain_logits(folder, dtype, history)[-1]))
        history.append(token)
        out.append(token)
    return out


def test_greedy_generation_through_the_entry_point(folders):
    """Prompts of 1 to 70 tokens in portions of 16, 20 greedy tokens each, float32: every token is the plain side's."""
    from sprout_lm_amd.engine import Engine
    for name in ("general", "odd", "states"):
        engine = Engine.from_folder(folders[name], "float32", block_size=MH.PAGE[name], num_blocks=64, max_sequences=4,
                                    max_batch_tokens=48, prefill_chunk_size=16, record_trace=True)
        vocab = MH.CONFIGS[name]["vocab"]
        prompts = [MH.random_tokens(vocab, n, 40 + i) for i, n in enumerate((1, 9, 40, 70))]
        outputs = engine.generate(prompts, max_new_tokens=20, ignore_eos=True)
        for prompt, got in zip(prompts, outputs):
            assert got == plain_greedy(folders[name], "float32", prompt, 20), f"{name}, prompt of {len(prompt)}"
        assert all(free == g.pool.num_pages for free, g in zip(engine.cache.free_pages(), engine.cache.groups))


def test_scheduling_never_changes_generation(folders):
    """Too few pages (preemption: the state slot is given back, then the prompt and what was generated are computed again
    from a cleared slot) and a late arrival give what each request generates alone."""
    from sprout_lm_amd.engine import Engine
    name, dtype = "general", "float32"
    vocab = MH.CONFIGS[name]["vocab"]
    prompts = {"A": MH.random_tokens(vocab, 33, 78), "B": MH.random_tokens(vocab, 29, 79),
               "C": MH.random_tokens(vocab, 40, 80), "D": MH.random_tokens(vocab, 3, 81)}
    want = {k: plain_greedy(folders[name], dtype, p, 14) for k, p in prompts.items()}
    for num_blocks, expect_preemption in ((64, False), (12, True)):
        engine = Engine.from_folder(folders[name], dtype, block_size=8, num_blocks=num_blocks, max_sequences=4,
                                    max_batch_tokens=24, prefill_chunk_size=16, record_trace=True)
        engine.add("A", prompts["A"], 14, ignore_eos=True)
        engine.step(); engine.step(); engine.step()
        for k in "BCD":
            engine.add(k, prompts[k], 14, ignore_eos=True)
        ticks = 0
        while engine.pending:
            ticks += 1
            assert ticks < 2000
            engine.step()
        for k in prompts:
            assert engine.result(k)["output"] == want[k], f"request {k} with {num_blocks} pages"
        assert any(e["type"] == "preempted" for e in engine.trace) == expect_preemption


def test_recorded_steps_equal_eager_steps(folders):
    """Steps replayed from recorded graphs (decoded tokens with the sampler inside, portions of recurring shapes) give
    the tokens of eagerly launched steps: the states go through the graphs' buffers unharmed."""
    from sprout_lm_amd.engine import Engine
    name = "general"
    vocab = MH.CONFIGS[name]["vocab"]
    prompts = [MH.random_tokens(vocab, n, 60 + i) for i, n in enumerate((7, 21, 3, 40, 12))]

    def run(use_graphs):
        engine = Engine.from_folder(folders[name], "float32", block_size=16, num_blocks=48, max_sequences=4,
                                    max_batch_tokens=32, prefill_chunk_size=16)
        engine.model.use_graphs = use_graphs
        engine.add("r0", prompts[0], 30, ignore_eos=True)
        engine.add("r1", prompts[1], 25, ignore_eos=True)
        steps = 0
        while engine.pending:
            steps += 1
            if steps == 6:
                engine.add("r2", prompts[2], 20, temperature=0.8, seed=5, ignore_eos=True)
            if steps == 15:
                engine.add("r3", prompts[3], 10, ignore_eos=True)
                engine.add("r4", prompts[4], 28, temperature=1.2, seed=9, ignore_eos=True)
            engine.step()
        replays = engine.model._graphs.replays if engine.model._graphs else 0
        return [engine.result(f"r{i}")["output"] for i in range(5)], replays

    eager, none = run(False)
    graphed, replays = run(True)
    assert none == 0 and replays > 40
    assert graphed == eager


def test_command_line_generates(folders):
    done = subprocess.run([sys.executable, "-m", "sprout_lm_amd", "generate", folders["general"], "--prompt-ids",
                           "3,1,4,1,5,9,2,6", "--dtype", "float32", "--ignore-eos"], cwd=ROOT,
                          env=dict(os.environ, MAX_NEW_TOKENS="6"), capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr
    final = json.loads(done.stdout.strip().splitlines()[-1])
    assert final["output"] == plain_greedy(folders["general"], "float32", [3, 1, 4, 1, 5, 9, 2, 6], 6)
