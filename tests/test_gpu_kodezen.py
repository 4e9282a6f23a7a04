"""Kodezen on the GPU: every mechanism alone against its plain function, then whole models cut into steps in different
ways, then generation through the engine's entry point and scheduler."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from sprout_lm_amd.cache.spec import StateSpec
from tests import kodezen_helpers as KH
from tests import traces
from tests.plain import kodezen_plain as K
from tests.test_gpu_megozen import Harness, dev
from tests.test_gpu_morarax import close, rounded, run_in_portions, specs_of, store_of

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]
PORTIONS = [(16, 1), (5, 9), (1, 1), (2, 3), (13, 8), (1, 2), (40, 40), (1, 1), (1, 1), (250, 250)]


def weights_for(part, rng, dtype, given=None):
    out = {}
    for name, spec in part.tensors().items():
        a = KH.random_array(rng, "mix." + name, spec.shape) if name not in ("in", "q", "k", "o", "up", "down") \
            else rng.normal(0, 0.15, spec.shape)
        out[name] = rounded(a, dtype).reshape(spec.shape)
    out.update(given or {})
    return out


def bind(part, weights, dtype):
    part.bind({name: dev(a, dtype) for name, a in weights.items()})
    part.prepare(DEV, dtype)


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_with_weights_around_zero_and_scaled_embedding(dtype):
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(1)
    part = make_part("norm", "rmsnorm", size=100, eps=1e-3, tensor="norm1", one_plus=True)
    w = rounded(rng.normal(0, 0.1, 100), dtype)
    bind(part, {"norm1": w}, dtype)
    x = (rng.standard_normal((7, 100)) * rng.uniform(0.01, 30.0, (7, 1))).astype(np.float32)
    out = torch.empty(7, 100, dtype=dtype, device=DEV)
    part.forward(None, dev(x), out)
    close(out.float().cpu().numpy(), K.one_plus_norm(x, w, 1e-3), dtype, "norm", bf16=2.0 ** -7)
    table = rounded(rng.standard_normal((50, 36)), dtype)
    embed = make_part("embedding", "token_embedding", vocab=50, hidden=36, tensor="embed", scale=16.0)
    bind(embed, {"embed": table}, dtype)
    tokens = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    residual = torch.empty(4, 36, device=DEV)
    embed.forward(None, tokens, residual)
    assert np.array_equal(residual.cpu().numpy(), (table[[3, 49, 0, 3]] * 16.0).astype(np.float32))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("channels,taps,bias,act,residual", [(100, 3, False, None, True), (320, 4, True, "silu", False),
                                                             (36, 1, True, "silu", False), (64, 1, False, None, True),
                                                             (700, 7, False, None, False)])
def test_short_convolution_in_portions(dtype, channels, taps, bias, act, residual):
    """Two requests beside each other in portions from one token to 250: portions shorter than the convolution, single
    tokens, and the very first tokens (zeros before them)."""
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(channels + taps)
    part = make_part("conv", "short_conv", channels=channels, taps=taps, tensor="c", bias="c.b" if bias else None,
                     residual=residual, activation=act)
    w = {"c": rounded(rng.normal(0, 0.5, (channels, taps)), dtype)}
    if bias:
        w["c.b"] = rounded(rng.normal(0, 0.2, channels), dtype)
    bind(part, w, dtype)
    inputs = [rounded(rng.standard_normal((n, channels)), dtype) for n in (330, 316)]
    specs = [part.cache_spec()] if taps > 1 else [StateSpec((1,), "float32")]
    harness = Harness(specs, dtype, page=8, pages=8, slots=2)
    seqs = [harness.cache.create() for _ in inputs]
    fed = [0, 0]
    got = [np.zeros_like(x, dtype=np.float32) for x in inputs]
    for step in PORTIONS:
        batch = [(i, min(n, len(inputs[i]) - fed[i])) for i, n in enumerate(step) if fed[i] < len(inputs[i])]
        ctx, entries = harness.context([(seqs[i], [0] * n) for i, n in batch])
        x = torch.cat([dev(inputs[i][fed[i]:fed[i] + n], dtype) for i, n in batch])
        out = torch.empty_like(x)
        part.forward(ctx, x, out, harness.view(ctx, 0) if taps > 1 else None)
        harness.commit(entries)
        row = 0
        for i, n in batch:
            got[i][fed[i]:fed[i] + n] = out[row:row + n].float().cpu().numpy()
            fed[i] += n
            row += n
    for i, x in enumerate(inputs):
        y = K.causal_conv(x, w["c"], w.get("c.b"))
        if act:
            y = K.silu(y)
        if residual:
            y = y + x
        close(got[i], y, dtype, f"convolution, request {i}", bf16=2.0 ** -7)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,vdim,state,groups,taps,parts", [(3, 10, 5, 1, 2, 3), (4, 32, 64, 1, 4, 2), (8, 16, 128, 4, 3, 4),
                                                                (4, 6, 9, 2, 1, 1), (2, 64, 200, 2, 4, 1), (6, 32, 48, 3, 4, 3), (2, 32, 128, 1, 2, 1)])
def test_state_space_duality_alone_in_portions(dtype, heads, vdim, state, groups, taps, parts):
    from sprout_lm_amd.parts import make_part
    hidden, eps = 48, 1e-5
    rng = np.random.default_rng(heads * 100 + state)
    part = make_part("mixer", "state_space_duality", hidden=hidden, heads=heads, vdim=vdim, state=state, groups=groups, taps=taps,
                     norm_groups=parts, eps=eps)
    w = weights_for(part, rng, dtype)
    bind(part, w, dtype)
    inputs = [rounded(rng.standard_normal((n, hidden)), dtype) for n in (330, 316)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": taps, "norm_groups": parts}
    for i, x in enumerate(inputs):
        close(got[i], K.mamba2_mixer(w, "", m, x, eps, store_of(dtype)), dtype, f"request {i}", f32=3e-5, bf16=4e-2)


def test_a_slow_head_remembers_and_a_fast_head_forgets():
    """A head whose rate is almost zero still holds, 600 tokens later, what one early token wrote; a head with a large rate has
    lost it.  The early token alone drives B, and the last token alone reads with C."""
    from sprout_lm_amd.parts import make_part
    hidden, heads, vdim, state = 16, 2, 8, 8
    part = make_part("mixer", "state_space_duality", hidden=hidden, heads=heads, vdim=vdim, state=state, groups=1, taps=1,
                     norm_groups=2, eps=1e-6)
    inner = heads * vdim
    w = {name: np.zeros(spec.shape, np.float32) for name, spec in part.tensors().items()}
    w_in = w["in"]
    w_in[:inner, 0] = 4.0                      # z: an open gate for everyone
    w_in[inner:2 * inner, 1] = 1.0             # u from feature 1
    w_in[2 * inner:2 * inner + state, 2] = 1.0        # B from feature 2 (the early token)
    w_in[2 * inner + state:2 * inner + 2 * state, 3] = 1.0    # C from feature 3 (the reader)
    w["conv"][:] = 1.0
    w["A_log"][:] = (-14.0, 1.5)
    w["norm"][:] = 1.0
    w["o"][:] = np.random.default_rng(0).normal(0, 0.3, w["o"].shape)
    bind(part, w, torch.float32)
    x = np.zeros((640, hidden), np.float32)
    x[:, 0] = 1.0
    x[5, 1] = x[5, 2] = 3.0
    x[620, 3] = 3.0
    got = run_in_portions(part, specs_of(part), torch.float32, [x], [(7,), (300,), (1,), (200,), (132,)], hidden)[0]
    m = {"heads": heads, "vdim": vdim, "state": state, "groups": 1, "conv": 1, "norm_groups": 2}
    want = K.mamba2_mixer(w, "", m, x, 1e-6)
    close(got, want, torch.float32, "far token")
    gated = np.linalg.lstsq(w["o"].astype(np.float64), want[620], rcond=None)[0]
    assert np.abs(gated[:vdim]).max() > 0.5 and np.abs(gated[vdim:]).max() < 1e-3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("inner,state,rank,taps", [(36, 5, 3, 4), (256, 16, 8, 4), (20, 1, 1, 1), (64, 40, 16, 2), (200, 130, 9, 3),
                                                   (192, 20, 12, 3)])
def test_selective_scan_alone_in_portions(dtype, inner, state, rank, taps):
    from sprout_lm_amd.parts import make_part
    hidden = 48
    rng = np.random.default_rng(inner + state)
    part = make_part("mixer", "selective_scan", hidden=hidden, inner=inner, state=state, dt_rank=rank, taps=taps)
    w = weights_for(part, rng, dtype)
    bind(part, w, dtype)
    inputs = [rounded(rng.standard_normal((n, hidden)), dtype) for n in (330, 316)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    m = {"inner": inner, "state": state, "dt_rank": rank, "conv": taps}
    for i, x in enumerate(inputs):
        close(got[i], K.mamba1_mixer(w, "", m, x, store_of(dtype)), dtype, f"request {i}", f32=3e-5, bf16=4e-2)


def attention_part(hidden, heads, kv_heads, dim, scale, taps, rot_dims, base, mask, eps):
    from sprout_lm_amd.parts import make_part
    position = make_part("position", "rotary_interleaved", rotary_dim=rot_dims, theta=base) if rot_dims \
        else make_part("position", "none", head_dim=dim)
    return make_part("mixer", "mixed_heads_attention", hidden=hidden, heads=heads, kv_heads=kv_heads, dim=dim, scale=scale,
                     position=position, taps=taps, eps=eps, window=mask[0] if mask else None, keep_first=mask[1] if mask else 0)


def attention_sizes(heads, kv_heads, dim, scale, taps, rot_dims, base, mask):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale, "conv": taps,
         "rot": {"dims": rot_dims, "base": base}}
    if mask:
        m["mask"] = {"size": mask[0], "keep_first": mask[1]}
    return m


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,kv_heads,dim,taps,rot_dims,mask", [
    (6, 3, 12, 3, 8, (7, 2)), (3, 3, 20, 1, 0, None), (4, 1, 32, 4, 32, (24, 20)), (8, 4, 16, 2, 8, (64, 0)),
    (6, 3, 16, 2, 16, (1, 0)), (4, 2, 128, 3, 96, (48, 5)), (2, 1, 48, 1, 24, (300, 1)), (4, 2, 32, 2, 16, (20, 150)),
    (2, 1, 64, 1, 0, (10, 300))])
def test_attention_alone_in_portions(dtype, heads, kv_heads, dim, taps, rot_dims, mask):
    hidden, eps, scale, base = 40, 1e-5, 0.7 / np.sqrt(dim), 200.0
    rng = np.random.default_rng(heads * 10 + dim)
    part = attention_part(hidden, heads, kv_heads, dim, scale, taps, rot_dims, base, mask, eps)
    w = weights_for(part, rng, dtype, None)
    bind(part, w, dtype)
    inputs = [rounded(rng.standard_normal((n, hidden)), dtype) for n in (330, 316)]
    got = run_in_portions(part, specs_of(part), dtype, inputs, PORTIONS, hidden)
    m = attention_sizes(heads, kv_heads, dim, scale, taps, rot_dims, base, mask)
    for i, x in enumerate(inputs):
        want = K.attention_mixer(w, "", m, x, np.arange(len(x)), eps, store_of(dtype))
        close(got[i], want, dtype, f"request {i}", f32=3e-5, bf16=4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("page", [8, 16])
def test_attention_keys_at_the_window_s_edges_and_kept_first_keys(dtype, page):
    """One flagged key whose score towers over its row and whose value is far from the rest: just inside the window, just
    outside, the last kept first key, the first one not kept, far away, at a page's first and last place; the reader in a
    portion of a prompt and decoded alone.  One key too many or too few moves the output by the size of a value."""
    hidden, heads, kv_heads, dim, window, keep = 24, 4, 2, 16, 36, 5
    scale, eps = 2.0, 1e-6
    part = attention_part(hidden, heads, kv_heads, dim, scale, 1, 8, 100.0, (window, keep), eps)
    rng = np.random.default_rng(5)
    w = weights_for(part, rng, dtype)
    # feature 0 flags a key, feature 1 a reader: both point along the unturned dimensions 8..15 of every head
    for name, column, gain in (("k", 0, 6.0), ("q", 1, 6.0)):
        w[name] = (w[name] * 0.2).astype(np.float32)
        w[name].reshape(-1, dim, hidden)[:, 8:, column] = gain
        w[name] = rounded(w[name], dtype)
    w["q.conv"][:] = 1.0
    w["k.conv"][:] = 1.0
    bind(part, w, dtype)
    m = attention_sizes(heads, kv_heads, dim, scale, 1, 8, 100.0, (window, keep))
    n = 260
    for reader, key in ((200, 165), (200, 164), (200, 4), (200, 5), (200, 50), (227, 192), (227, 191), (96, 61), (91, 56),
                        (259, 0), (40, 4), (41, 5), (35, 0), (39, 3)):
        x = rounded(rng.standard_normal((n, hidden)) * 0.3, dtype)
        x[:, :2] = 0.0
        x[key, 0] = 4.0
        x[reader, 1] = 4.0
        want = K.attention_mixer(w, "", m, x, np.arange(n), eps, store_of(dtype))
        seen = key <= reader and (reader - key < window or key < keep)
        lone = K.attention_mixer(w, "", m, np.where(np.arange(n)[:, None] == key, 0.0, x), np.arange(n), eps, store_of(dtype))
        assert (np.abs(want[reader] - lone[reader]).max() > 0.5) == seen, (reader, key)
        for steps in ([(reader + 1,), (n,)], [(reader,), (1,), (n,)], [(33,), (reader - 33,), (1,), (1,), (n,)]):
            got = run_in_portions(part, specs_of(part), dtype, [x], steps, hidden, page=page)[0]
            close(got[reader], want[reader], dtype, f"reader {reader}, key {key}, steps {steps}", f32=3e-5, bf16=4e-2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,inner,T", [(100, 28, 7), (128, 96, 5), (128, 96, 70), (64, 64, 300)])
def test_dense_feed_forward_with_biases(dtype, hidden, inner, T):
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(hidden + T)
    part = make_part("feed_forward", "mlp", hidden=hidden, inner=inner, activation="gelu_erf", bias=".b")
    w = weights_for(part, rng, dtype)
    bind(part, w, dtype)
    x = rounded(rng.standard_normal((T, hidden)), dtype)
    harness = Harness([StateSpec((1,), "float32")], dtype)
    ctx, _ = harness.context([(harness.cache.create(), [0] * T)])
    residual = torch.zeros(T, hidden, device=DEV)
    part.forward(ctx, dev(x, dtype), residual)
    close(residual.cpu().numpy(), K.dense_ff(w, "", x, store_of(dtype)), dtype, "dense feed-forward")
    # from the residual stream, the norm folded into the first product where a kernel does that (few tokens, bfloat16)
    norm = make_part("norm", "rmsnorm", size=hidden, eps=1e-5, tensor="n", one_plus=True)
    nw = rounded(rng.normal(0, 0.1, hidden), dtype)
    bind(norm, {"n": nw}, dtype)
    stream = (rng.standard_normal((T, hidden)) * 3.0).astype(np.float32)
    residual = dev(stream)
    if part.forward_from_residual(ctx, norm, residual):
        want = stream + K.dense_ff(w, "", store_of(dtype)(K.one_plus_norm(stream, nw, 1e-5)), store_of(dtype))
        close(residual.cpu().numpy(), want, dtype, "dense feed-forward from the residual")
        print(f"norm folded into the product: hidden {hidden}, inner {inner}, {T} tokens")


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,inner,experts,top,T", [(100, 12, 5, 2, 9), (128, 64, 4, 1, 70), (64, 32, 8, 8, 33), (128, 80, 8, 1, 300),
                                                        (256, 80, 6, 3, 1)])
def test_routed_experts_weighted_on_their_input(dtype, hidden, inner, experts, top, T):
    """Sigmoid scores, the largest chosen, no renormalising, the weight on what the expert reads: silu is not linear, so a
    weight on the output instead shows."""
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(hidden + experts + T)
    part = make_part("feed_forward", "routed_experts", hidden=hidden, inner=inner, experts=experts, top=top, router_bias=False,
                     routing="sigmoid_top", weight_on="input")
    w = {name: rounded(rng.normal(0, 0.5 if name == "router" else 0.15, spec.shape), dtype) for name, spec in part.tensors().items()}
    bind(part, dict(w), dtype)
    x = rounded(rng.standard_normal((T, hidden)), dtype)
    harness = Harness([StateSpec((1,), "float32")], dtype)
    ctx, _ = harness.context([(harness.cache.create(), [0] * T)])
    residual = torch.zeros(T, hidden, device=DEV)
    part.forward(ctx, dev(x, dtype), residual)
    want = K.routed_ff(w, "", {"router": {"experts": experts, "top": top}}, x, store_of(dtype))
    close(residual.cpu().numpy(), want, dtype, "routed feed-forward", bf16=3e-2)


# ---------------------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("kodezen"))
    return {name: KH.make_folder(root, name) for name in KH.CONFIGS}


def requests_for(name, lengths, seed=100):
    vocab = KH.CONFIGS[name]["vocab"]
    return {f"r{i}": KH.random_tokens(vocab, n, seed + i) for i, n in enumerate(lengths)}


def replay(folder, name, dtype, trace, max_tokens, page=None, slots=4, reused=None):
    """The engine's trace session on a pool of `max_tokens`; per step the logits rows."""
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.trace import TraceSession
    page = page or KH.PAGE[name]
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
            want = KH.plain_logits(folder, dtype, requests[rid])[pos]
            err = float(np.abs(got[i] - want).max())
            worst = max(worst, err)
            bound = KH.tolerance(dtype, want)
            if dtype == "bfloat16":     # how far bfloat16 rounding moves this row on the plain side itself
                bound += float(np.abs(want - KH.plain_logits(folder, "float32", requests[rid])[pos]).max())
            assert err <= bound, f"step {step} request {rid} position {pos}: error {err:.3e}"
    return worst


LENGTHS = {"odd": [1, 2, 21, 70, 45, 97], "general": [1, 9, 40, 97, 150, 33, 2, 75], "states": [9, 40, 97, 33, 130, 3],
           "attention": [2, 70, 97, 33, 64, 120]}
CASES = [(n, "float32") for n in KH.CONFIGS] + [(n, "bfloat16") for n in KH.CONFIGS]


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
    """Prompts of 700 tokens whole, in long uneven portions, and two requests' long portions beside each other and beside
    single tokens: windows pass pages by the dozen while the first keys stay."""
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


def test_a_window_gives_pages_back_but_not_the_first(folders):
    """A request far longer than the pool: the window's pages are used again and again, the pages of the kept first keys
    never, and every row still agrees with the plain side, which keeps everything."""
    name, dtype = "general", "float32"      # windows of 24 (20 kept: two pages of 16) and 64
    requests = requests_for(name, [600], seed=900)
    trace = traces.portions(requests, sizes=(50, 1, 1, 33, 2, 70))
    results = replay(folders[name], name, dtype, trace, 192)      # 12 pages a group for 600 tokens
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
        tokens = KH.random_tokens(KH.CONFIGS[name]["vocab"], 260, 9)
        runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=40, max_sequences=2,
                                         prefix_caching=False)
        seq = runner.cache.create()
        want = KH.plain_logits(folders[name], dtype, tokens)
        for p, token in enumerate(tokens):
            assert runner.cache.reserve(seq, p + 1)
            got = runner.step([StepEntry(seq, [token], [0])]).cpu().numpy()[0]
            assert np.abs(got - want[p]).max() <= KH.tolerance(dtype, want[p]), f"{name} {dtype} position {p}"
        seq.release()


def test_a_state_slot_starts_from_zero_again(folders):
    """A request that takes over the slot of a finished one computes what it computes on a fresh engine."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    name, dtype = "states", "float32"
    runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=16, max_sequences=1, prefix_caching=False)
    vocab = KH.CONFIGS[name]["vocab"]
    for seed in (1, 2, 3):
        tokens = KH.random_tokens(vocab, 50, seed)
        seq = runner.cache.create()
        assert seq.state_slot == 0 and runner.cache.reserve(seq, 50)
        got = runner.step([StepEntry(seq, tokens, [49])]).cpu().numpy()[0]
        want = KH.plain_logits(folders[name], dtype, tokens)[49]
        assert np.abs(got - want).max() <= KH.tolerance(dtype, want)
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
    vocab = KH.CONFIGS[name]["vocab"]
    results = [np.fromfile(out / f"{r['step']}.f32", dtype="<f4").reshape(len(rows), vocab) if rows else None
               for r, rows in zip(trace.steps, trace.expected)]
    check(folders[name], dtype, requests, trace, results)


# ---------------------------------------------------------------------------------------------- generation
def plain_greedy(folder, dtype, prompt, steps):
    history, out = list(prompt), []
    for _ in range(steps):
        token = int(np.argmax(KH.plain_logits(folder, dtype, history)[-1]))
        history.append(token)
        out.append(token)
    return out


def test_greedy_generation_through_the_entry_point(folders):
    """Prompts of 1 to 70 tokens in portions of 16, 20 greedy tokens each, float32: every token is the plain side's."""
    from sprout_lm_amd.engine import Engine
    for name in ("general", "odd", "states"):
        engine = Engine.from_folder(folders[name], "float32", block_size=KH.PAGE[name], num_blocks=64, max_sequences=4,
                                    max_batch_tokens=48, prefill_chunk_size=16, record_trace=True)
        vocab = KH.CONFIGS[name]["vocab"]
        prompts = [KH.random_tokens(vocab, n, 40 + i) for i, n in enumerate((1, 9, 40, 70))]
        outputs = engine.generate(prompts, max_new_tokens=20, ignore_eos=True)
        for prompt, got in zip(prompts, outputs):
            assert got == plain_greedy(folders[name], "float32", prompt, 20), f"{name}, prompt of {len(prompt)}"
        assert all(free == g.pool.num_pages for free, g in zip(engine.cache.free_pages(), engine.cache.groups))


def test_scheduling_never_changes_generation(folders):
    """Too few pages (preemption: the state slot is given back, then the prompt and what was generated are computed again
    from a cleared slot) and a late arrival give what each request generates alone."""
    from sprout_lm_amd.engine import Engine
    name, dtype = "attention", "float32"      # its last layer has no window: its pages are never given back
    vocab = KH.CONFIGS[name]["vocab"]
    prompts = {"A": KH.random_tokens(vocab, 33, 78), "B": KH.random_tokens(vocab, 29, 79),
               "C": KH.random_tokens(vocab, 40, 80), "D": KH.random_tokens(vocab, 3, 81)}
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
    vocab = KH.CONFIGS[name]["vocab"]
    prompts = [KH.random_tokens(vocab, n, 60 + i) for i, n in enumerate((7, 21, 3, 40, 12))]

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
