"""Zeganex on the GPU against the plain implementation (tests/plain_zeganex.py): every mechanism alone,
whole prompts, token-by-token decoding, portions, mixed batches with pages and state slots used again,
tokens made to stand out at the places where a cache or a window can lose them, long decoding, and greedy
generation through the entry point."""
import copy
import random

import numpy as np
import pytest
import torch

from tests import plain_zeganex as P
from tests.helpers import steps_portions, steps_prefill_then_decode, steps_whole
from tests.samovik_helpers import rel_error, run_steps
from tests.test_samovik_gpu import mixed_steps
from tests.tumitar_helpers import run_steps_with_routes
from tests.zeganex_helpers import (CFG_A, CFG_B, CFG_C, CONFIGS, YARN, _dense, _moe, _rotary, _two_maps, build, one_layer,
                                   random_config, routed_layers, typed)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
# Of the logits' own root mean square.  Every branch output is normed to unit size before it joins the stream, so the
# rounding of a narrow random model is not damped on its way through the layers (a subtraction of two rounded maps,
# normed again, among it); every case that bfloat16 runs, float32 runs too, at a thousandth of the limit.
LIMIT = {"float32": 2e-5, "bfloat16": 6e-2}


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def run_and_check(model, steps, cfg, w, reqs, dtype, what="", **kw):
    """Run the steps and hold every position against the plain implementation.  In float32 the plain run routes
    by itself.  In bfloat16 a router's close call may fall the other way and then changes every later position
    through the caches: there the plain run is told which experts the framework chose, and every such choice
    must be one whose share of the router's softmax is within 0.02 of the plain run's own choice."""
    if dtype == "float32":
        got, routes = run_steps(model, steps, **kw), {}
    else:
        got, routes = run_steps_with_routes(model, steps, **kw)
    layers = routed_layers(cfg)
    for rid, toks in reqs.items():
        forced = None
        if routes.get(rid):
            assert len(routes[rid]) == len(layers), f"{what}: the framework routed in {len(routes[rid])} layers, the model has {len(layers)}"
            forced = {layer: r.long() for layer, r in zip(layers, routes[rid])}
        want = P.forward(w, cfg, toks, forced=forced).numpy()
        if forced:
            own = _own_routes(w, cfg, toks, forced)
            assert own < 0.02, f"{what}: request {rid}: an expert whose share is {own:.3f} under the router's own choice was taken"
        rows = got[rid]
        assert sorted(rows) == list(range(len(toks))), f"{what}: {rid} is missing positions"
        errs = {p: rel_error(rows[p], want[p]) for p in rows}
        first_bad = next((p for p in sorted(rows) if not errs[p] <= LIMIT[dtype]), None)
        assert first_bad is None, (f"{what} {dtype}: request {rid}: first wrong position {first_bad} of {len(toks)}, "
                                   f"worst error {max(errs.values()):.3e}")


def _own_routes(w, cfg, toks, forced) -> float:
    """How far under the plain router's own choice the forced experts' shares lie at worst, with the forced
    run's inputs (the stream that the forced choices lead to)."""
    worst = 0.0
    keep = []
    P.forward(w, cfg, toks, keep_layers=keep, forced=forced)
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    mem = P.SequenceMemory(cfg)
    x = P.embed(w, cfg, list(toks))
    pos = torch.arange(len(toks))
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = P.rms_norm(x, w[p + "norm1"], eps)
        shared = mem.layers[m["kv_from"]] if m.get("kv_from") is not None else None
        if layer["type"] == "attention":
            y = P.differential_attention(h, w, p + "mix.", m, pos, eps, mem.layers[i], shared)
        else:
            y = P.gated_rotary_attention(h, w, p + "mix.", m, pos, mem.layers[i], shared)
        x = x + mult * P.rms_norm(y, w[p + "norm1b"], eps)
        if i in forced:
            h = P.rms_norm(x, w[p + "norm2"], eps)
            scores = torch.softmax(h @ w[p + "mlp.router"].T, dim=-1)
            top = forced[i].shape[1]
            own = torch.topk(scores, top, dim=-1).values.min(dim=-1).values
            took = scores.gather(1, forced[i]).min(dim=-1).values
            worst = max(worst, float((own - took).max()))
        x = keep[i]
    return worst


def _session(model, page=16, blocks=64, slots=4):
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.runner import ModelRunner
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page, num_blocks=blocks,
                         max_requests=slots, dtype=model.dtype, device=DEV, input_state_need=model.input_state_need())
    return cache, ModelRunner(model, cache)


def _step_context(cache, runner, portions, tokens=None):
    """``portions``: (request, first position, count).  Returns the step's context and cache views."""
    from tensorline_amd.engine.batch import StepEntry
    entries = []
    for rid, lo, n in portions:
        if not cache.has_request(rid):
            cache.add_request(rid)
        cache.grow(rid, lo + n)
        entries.append(StepEntry(rid, list(tokens[rid][lo:lo + n]) if tokens else [0] * n, lo, [0]))
    packed = runner.pack(entries)
    return runner.context(packed, runner._upload(packed.data))


def _rms_error(got, want):
    return ((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item()


# ---- every mechanism alone -------------------------------------------------------------------------
def test_bigram_embedding_keeps_the_token_before_across_steps_and_slots():
    cfg = one_layer("attention_2", _rotary(1, 1, 8, 8, 1, 4, 0), width=40, vocab=90, bigram=(100003, 1000003, 19))
    model, w = build(cfg, "bfloat16", seed=2)
    cache, runner = _session(model, slots=2)
    toks = {"a": tokens_for(cfg, 30, 1), "b": tokens_for(cfg, 9, 2), "c": tokens_for(cfg, 5, 3)}
    want = {r: P.embed(w, cfg, t) for r, t in toks.items()}
    at = {r: 0 for r in toks}

    def step(portions):
        ctx, _ = _step_context(cache, runner, [(r, at[r], n) for r, n in portions], toks)
        got = model.embedding.forward_step(ctx).cpu()
        row = 0
        for r, n in portions:
            assert torch.equal(got[row:row + n], want[r][at[r]:at[r] + n]), f"{r} at {at[r]}, {n} tokens"
            row, at[r] = row + n, at[r] + n
    step([("a", 1), ("b", 4)])
    step([("a", 2)])
    step([("b", 1), ("a", 1)])
    step([("a", 20), ("b", 4)])
    cache.release("b")
    step([("c", 1), ("a", 1)])          # c takes b's slot; its first token reads the last row, not what b left
    step([("c", 4), ("a", 5)])


@pytest.mark.parametrize("case", [
    # query heads, key heads, dim, value heads, vdim, rotated dims, taps
    (4, 2, 24, 2, 40, 8, 3), (8, 4, 16, 2, 24, 0, 4), (3, 1, 10, 1, 7, 10, 1), (2, 2, 128, 2, 64, 32, 5), (3, 0, 6, 0, 9, 2, 2),
    (1, 1, 5, 1, 3, 4, 2)])
def test_convolution_rotation_and_cache_write_in_one_pass(case):
    """Portions shorter than the taps reach back, a sequence's first token, two sequences in a step, one-token steps
    (which renew the kept inputs in the same launch), a slot that another request used before: queries against the
    plain convolution and rotation, and what lies in the cache pages afterwards."""
    from tensorline_amd.ops import kernels
    from tensorline_amd.parts.rotary import yarn_frequencies
    Hq, Gk, d, Gv, dv, rot, K = case
    rep = Gk // Gv if Gv else 1
    D = -(-max(d, dv) // 16) * 16
    C = (Hq + Gk) * d + Gv * dv
    torch.manual_seed(sum(case))
    taps = torch.randn(C, K)
    freq, mag = yarn_frequencies(rot, 300.0, YARN) if rot else (None, 1.0)
    rotd = {"dims": rot, "base": 300.0, "scaling": YARN} if rot else None
    mixer = _rotary(max(Gk, 1), max(Gk, 1), D, D, K, 0, 0)                    # only for a cache of the right shape
    cfg = one_layer("attention_2", mixer, width=16)
    model, _ = build(cfg, "float32", seed=0)
    cache, runner = _session(model, slots=2)
    state = torch.zeros(3, max((K - 1) * C, 1) + 5, device=DEV)
    xs = {"a": torch.randn(30, C + 3), "b": torch.randn(12, C + 3)}
    want = {}
    for r, x in xs.items():
        y = P.short_conv(x[:, :C], taps)[0]
        pos = torch.arange(x.shape[0])
        q = P.rotate_pairs(y[:, :Hq * d].reshape(-1, Hq, d), pos, rotd)
        k = P.rotate_pairs(y[:, Hq * d:(Hq + Gk) * d].reshape(-1, Gk, d), pos, rotd) if Gk else None
        want[r] = (q, k, y[:, (Hq + Gk) * d:].reshape(-1, Gv, dv) if Gv else None)
    planes = cache.storage(0)
    keys, values = (planes["k"], planes["v"]) if Gk else (None, None)
    ctx, views = _step_context(cache, runner, [("old", 0, 9)])                # leaves its inputs in slot 0 ...
    kernels.conv_rotate_store(torch.randn(9, C, device=DEV), taps.t().contiguous().to(DEV), ctx, state, 5, freq.to(DEV) if rot else None, mag, keys,
                              values, views[0].slots if Gk else None, Hq, Gk, d, Gv, dv, D, rep, torch.float32)
    cache.release("old")                                                      # ... which "a" gets: the test zeroes it as the manager does
    state.zero_()
    at = {"a": 0, "b": 0}
    slots_of = {"a": [], "b": []}
    for step in ([("a", 1), ("b", 5)], [("a", 2)], [("a", 1), ("b", 1)], [("b", 2), ("a", 19)], [("a", 1)], [("a", 6), ("b", 4)]):
        ctx, views = _step_context(cache, runner, [(r, at[r], n) for r, n in step])
        x = torch.cat([xs[r][at[r]:at[r] + n] for r, n in step]).to(DEV)
        got = kernels.conv_rotate_store(x, taps.t().contiguous().to(DEV), ctx, state, 5, freq.to(DEV) if rot else None, mag, keys, values,
                                        views[0].slots if Gk else None, Hq, Gk, d, Gv, dv, D, rep, torch.float32).cpu()
        got = got.view(-1, Hq, D)
        row = 0
        for r, n in step:
            assert torch.allclose(got[row:row + n, :, :d], want[r][0][at[r]:at[r] + n], atol=2e-5), f"{r} at {at[r]}, {n} tokens"
            assert not got[row:row + n, :, d:].any()
            if Gk:
                slots_of[r] += views[0].slots[row:row + n].tolist()
            row, at[r] = row + n, at[r] + n
    assert at == {"a": 30, "b": 12}
    assert not state[:, :5].any()                                             # what lies ahead of the kept inputs is not touched
    if Gk:
        page = keys.shape[1]
        for r in xs:
            sl = torch.tensor(slots_of[r])
            k = keys.view(-1, Gk, D)[sl.to(DEV)].cpu()
            assert torch.allclose(k[:, :, :d], want[r][1], atol=2e-5) and not k[:, :, d:].any()
            v = values[(sl // page).to(DEV), :, :, (sl % page).to(DEV)].cpu()              # [tokens, Gk, D]
            for g in range(Gv):
                for m in range(rep):
                    assert torch.allclose(v[:, g * rep + m, :dv], want[r][2][:, g], atol=1e-6)


def test_two_maps_put_together_and_normed():
    from tensorline_amd.ops import kernels
    for H, G, dv, D, dtype in ((4, 2, 24, 32, torch.float32), (6, 1, 64, 64, torch.bfloat16), (3, 3, 7, 16, torch.float32), (2, 1, 200, 208, torch.float32)):
        torch.manual_seed(H)
        R = H // G
        a = torch.randn(5, G, 2, R, D).to(dtype)
        got = kernels.diff_combine(a.view(5, -1).to(DEV), H, G, dv, D, 0.37, 1e-5, 0.45).float().cpu().view(5, G, R, dv)
        o = a[:, :, 0, :, :dv].float() - 0.37 * a[:, :, 1, :, :dv].float()
        want = P.rms_divide(o, 1e-5) * 0.45
        assert torch.allclose(got, want, atol=1e-5 if dtype == torch.float32 else 2e-2)


def test_normed_branch_joins_the_stream_in_the_next_norm():
    from tensorline_amd.ops import kernels
    for H in (96, 50, 3, 4100):
        torch.manual_seed(H)
        x, y = torch.randn(7, H), torch.randn(7, H) * 3
        wb, wn = torch.randn(H), torch.randn(H)
        x2 = x + 0.45 * P.rms_norm(y, wb, 2e-5)
        branch = kernels.NormedBranch(y.to(DEV), wb.to(DEV), 2e-5, 0.45)
        xd = x.to(DEV)
        rows = torch.tensor([5, 0, 5], dtype=torch.int32, device=DEV)
        picked = kernels.add_rmsnorm(xd, branch, wn.to(DEV), 1e-6, torch.float32, rows=rows).cpu()
        assert torch.equal(xd.cpu(), x) and torch.allclose(picked, P.rms_norm(x2, wn, 1e-6)[[5, 0, 5]], atol=1e-5)
        out = kernels.add_rmsnorm(xd, branch, wn.to(DEV), 1e-6, torch.float32).cpu()
        assert torch.allclose(xd.cpu(), x2, atol=1e-5) and torch.allclose(out, P.rms_norm(x2, wn, 1e-6), atol=1e-5)
        xd = x.to(DEV)
        kernels.add_normed_branch(xd, branch)
        assert torch.allclose(xd.cpu(), x2, atol=1e-5)


def test_router_weighs_by_the_softmax_over_all_experts():
    from tensorline_amd.ops import kernels
    z = torch.tensor([[0.5, 3.0, -1.0, 3.0, 2.0], [-4.0, -9.0, -2.0, -3.0, -8.0]], device=DEV)
    ids, wts = kernels.moe_route(z, 3, "softmax_all")
    assert ids.tolist() == [[1, 3, 4], [2, 3, 0]]              # equal logits: the lower index first
    for r in range(2):
        assert torch.allclose(wts[r], torch.softmax(z[r], 0)[ids[r].long()], atol=1e-6)
    assert float(wts[0].sum()) < 1.0                            # nothing is renormalised
    z = torch.randn(9, 200, device=DEV)                         # more experts than a wave has lanes
    ids, wts = kernels.moe_route(z, 5, "softmax_all")
    want = torch.topk(torch.softmax(z, -1), 5)
    assert torch.equal(ids.long(), want.indices) and torch.allclose(wts, want.values, atol=1e-6)


MIXERS = [
    ("attention_2", _rotary(4, 2, 24, 40, 3, 21, 8, scaling=YARN)),
    ("attention_2", _rotary(1, 1, 10, 7, 1, 3, 10, base=20.0)),                    # all sizes odd or small, one tap, full rotation
    ("attention_2", _rotary(6, 1, 64, 64, 4, 40, 32, scaling=YARN)),               # matrix-core attention
    ("attention_2", _rotary(2, 2, 128, 32, 2, 0, 0, scale=0.03)),                   # no rotation, no window, values under the key size
    ("attention_2", _rotary(18, 2, 32, 48, 5, 100, 2)),                            # nine query heads a group
    ("attention", _two_maps(4, 2, 16, 24, 4, 33)),
    ("attention", _two_maps(1, 1, 10, 7, 1, 4, diff=0.9, scale=0.5)),
    ("attention", _two_maps(6, 2, 32, 64, 3, 17, diff=0.2)),                       # matrix-core attention, head size 64
    ("attention", _two_maps(2, 1, 128, 128, 2, 0, diff=0.5, scale=0.04)),
    ("attention", _two_maps(9, 3, 64, 16, 6, 70, diff=0.35, scale=0.1)),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(MIXERS)))
def test_mixer_alone(case, dtype):
    """Three sequences in one batch, each from its first token, then each continued by a second step of other
    sizes (one token among them): the mixer's outputs against the plain ones of the whole sequences."""
    kind, mixer = MIXERS[case]
    cfg = one_layer(kind, mixer, width=72)
    model, w = build(cfg, dtype, seed=case)
    first, second = [37, 1, 150], [1, 20, 3]
    torch.manual_seed(case)
    hs = [torch.randn(a + b, 72).to(torch.bfloat16).float() for a, b in zip(first, second)]

    def fn(x):
        pos = torch.arange(x.shape[0])
        if kind == "attention":
            return P.differential_attention(x, w, "l0.mix.", mixer, pos, 1e-6, P.MixerMemory())
        return P.gated_rotary_attention(x, w, "l0.mix.", mixer, pos, P.MixerMemory())
    cache, runner = _session(model)
    mix = model.blocks[0].mixer
    ctx, views = _step_context(cache, runner, [(i, 0, n) for i, n in enumerate(first)])
    got1 = mix.forward(torch.cat([h[:n] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    ctx, views = _step_context(cache, runner, [(i, a, b) for i, (a, b) in enumerate(zip(first, second))])
    got2 = mix.forward(torch.cat([h[n:] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    at1 = at2 = 0
    for h, a, b in zip(hs, first, second):
        want = fn(h)
        got = torch.cat((got1[at1:at1 + a], got2[at2:at2 + b]))
        err = _rms_error(got, want)
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{kind} {mixer}: sequence of {a} + {b}: {err:.3e}"
        at1, at2 = at1 + a, at2 + b


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mlp", [_dense(136), _dense(7), _moe(6, 2, 40), _moe(3, 3, 20), _moe(1, 1, 100), _moe(40, 5, 16)])
def test_feed_forward_alone(mlp, dtype):
    """Few rows and many (the grouped product's tiles of 16 and of 64 rows)."""
    cfg = one_layer("attention_2", _rotary(1, 1, 8, 8, 1, 4, 0), mlp, width=88)
    model, w = build(cfg, dtype, seed=3)
    ff = model.blocks[0].feed_forward
    for rows in (1, 5, 300):
        torch.manual_seed(rows)
        h = (torch.randn(rows, 88) * 2).to(torch.bfloat16).float()
        got = ff.forward(h.to(DEV).to(model.dtype), None).float().cpu()
        want = P.dense_feed_forward(h, w, "l0.mlp.") if mlp["kind"] == "dense" else P.routed_feed_forward(h, w, "l0.mlp.", mlp)
        err = (got - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{rows} rows: {err:.3e}"


# ---- a token made loud: what a wrong window, a lost page or a lost kept input would show ------------------------
def _loud_case(kind, window, page):
    if kind == "attention":
        return _two_maps(4, 2, 32, 64, 3, window, diff=0.4, scale=0.3)
    return _rotary(4, 2, 64, 64, 3, window, 16, scale=0.2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
@pytest.mark.parametrize("window", [37, 48, 200])
def test_a_loud_token_at_the_edges_of_window_and_pages(kind, window, dtype):
    """One input row of the mixer is made twenty-five times as large as the others, so that its key takes nearly all the
    weight of the queries it agrees with and its value dominates what they read: whether it is seen shows in every
    output around it.  It sits at the sequence's first token, at both sides of a page's border, and hundreds of
    tokens back; outputs are compared just inside and just outside the window (and the taps' reach beyond it),
    computed as part of a prompt, of portions cut at the edge, and decoded one by one."""
    mixer = _loud_case(kind, window, 16)
    cfg = one_layer(kind, mixer, width=64)
    model, w = build(cfg, dtype, seed=9)
    mix = model.blocks[0].mixer
    n = 300
    for loud in (0, 15, 16, 31, 290 - window):
        torch.manual_seed(loud)
        h = torch.randn(n, 64)
        h[loud] *= 25.0
        h = h.to(torch.bfloat16).float()
        pos = torch.arange(n)
        if kind == "attention":
            want = P.differential_attention(h, w, "l0.mix.", mixer, pos, 1e-6, P.MixerMemory())
            quiet = P.differential_attention(torch.cat((h[:loud], h[loud:loud + 1] / 25.0, h[loud + 1:])), w, "l0.mix.", mixer, pos,
                                             1e-6, P.MixerMemory())
        else:
            want = P.gated_rotary_attention(h, w, "l0.mix.", mixer, pos, P.MixerMemory())
            quiet = P.gated_rotary_attention(torch.cat((h[:loud], h[loud:loud + 1] / 25.0, h[loud + 1:])), w, "l0.mix.", mixer, pos,
                                             P.MixerMemory())
        last_in = min(loud + window - 1, n - 1)
        assert _rms_error(quiet[last_in:last_in + 1], want[last_in:last_in + 1]) > 0.1, "the loud token does not show at the window's edge"
        edge = loud + window
        cuts = {"whole": [n], "cut at the edge": [min(edge, n - 2), 2, n], "decoded across the edge": [max(min(edge - 3, n - 8), 1)] + [1] * 8 + [n]}
        for name, sizes in cuts.items():
            cache, runner = _session(model, blocks=40)
            got, at = [], 0
            for size in sizes:
                size = min(size, n - at)
                if size <= 0:
                    break
                ctx, views = _step_context(cache, runner, [("a", at, size)])
                got.append(mix.forward(h[at:at + size].to(DEV).to(model.dtype), ctx, views[0]).float().cpu())
                at += size
                cache.trim("a", at)
            got = torch.cat(got)
            assert at == n
            tol = 1e-5 if dtype == "float32" else 4e-2
            for lo, hi in ((0, n), (max(edge - 2, 0), min(edge + 4, n))):
                if lo < hi:
                    err = _rms_error(got[lo:hi], want[lo:hi])
                    assert err < tol, f"{kind} window {window}, loud token at {loud}, {name}: positions {lo}..{hi}: {err:.3e}"


# ---- whole models in the cuttings ----------------------------------------------------------------------
CUTS = {"whole": steps_whole, "decode": lambda r: steps_prefill_then_decode(r, tail=9), "portions": steps_portions}


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("cut", list(CUTS))
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_cuttings_against_plain(name, cut, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=11)
    reqs = {"x": tokens_for(cfg, 75, 1), "y": tokens_for(cfg, 1, 2), "z": tokens_for(cfg, 34, 3)}
    run_and_check(model, CUTS[cut](reqs), cfg, w, reqs, dtype, f"{name} {cut}", page_size=16 if name != "B" else 8, max_tokens=128)


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_down_to_two_tokens_and_one(dtype):
    cfg = CFG_A
    model, w = build(cfg, dtype, seed=4)
    reqs = {"x": tokens_for(cfg, 61, 5)}
    for sizes in ((2,), (1,), (2, 1, 3), (17, 2, 2, 1, 30)):
        run_and_check(model, steps_portions(reqs, sizes=sizes), cfg, w, reqs, dtype, f"portions of {sizes}", max_tokens=128)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(name, dtype):
    cfg = CONFIGS[name]
    model, w = build(cfg, dtype, seed=12)
    rng = random.Random(5)
    reqs = {f"r{i}": tokens_for(cfg, n, 20 + i) for i, n in enumerate([50, 3, 33, 1, 64, 17, 48, 2, 31])}
    # a pool that holds four live requests and no more: every page and slot is handed out several times
    run_and_check(model, mixed_steps(reqs, rng), cfg, w, reqs, dtype, f"{name} mixed", page_size=16, max_tokens=4 * 64, max_requests=4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_request_alone_and_in_a_batch_of_unequal_requests(dtype):
    cfg = CFG_C
    model, w = build(cfg, dtype, seed=14)
    reqs = {"a": tokens_for(cfg, 90, 1), "b": tokens_for(cfg, 7, 2), "c": tokens_for(cfg, 41, 3)}
    alone = {r: run_steps(model, steps_portions({r: t}, sizes=(30, 1, 11)), max_tokens=256)[r] for r, t in reqs.items()}
    steps, at = [], {r: 0 for r in reqs}
    sizes = {"a": (30, 1, 11), "b": (2, 1), "c": (5, 25, 1)}
    k = 0
    while any(at[r] < len(reqs[r]) for r in reqs):
        entries, end = [], []
        for r, t in reqs.items():
            if at[r] < len(t):
                n = min(sizes[r][k % len(sizes[r])], len(t) - at[r])
                entries.append({"id": r, "tokens": t[at[r]:at[r] + n], "want": list(range(n))})
                at[r] += n
                if at[r] == len(t):
                    end.append(r)
        steps.append({"entries": entries, "end": end})
        k += 1
    together = run_steps(model, steps, max_tokens=256)
    tol = 1e-5 if dtype == "float32" else LIMIT[dtype]
    for r, t in reqs.items():
        for p in range(len(t)):
            assert rel_error(together[r][p], alone[r][p]) < tol, f"{r} at {p}: the batch changes a request's logits"


def test_the_first_tokens_and_a_slot_used_again():
    """A request of one token, then one of two, then one decoded from its first token on, all through one state
    slot: nothing of an earlier request (its kept inputs, its last token, its pages) reaches the next."""
    cfg = CFG_A
    model, w = build(cfg, "float32", seed=6)
    reqs = {"p": tokens_for(cfg, 1, 1), "q": tokens_for(cfg, 2, 2), "r": tokens_for(cfg, 40, 3), "s": tokens_for(cfg, 5, 4)}
    steps = steps_whole({"p": reqs["p"], "q": reqs["q"]}) + steps_portions({"r": reqs["r"]}, sizes=(1,)) + steps_whole({"s": reqs["s"]})
    run_and_check(model, steps, cfg, w, reqs, "float32", "first tokens", max_tokens=64, max_requests=1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_tokens_far_back_reach_the_end_through_the_layers(dtype):
    """Windows of 40 and 64 in four layers and taps of four reach back a few hundred tokens: the first tokens of a
    400-token prompt still show at its end when it is computed in portions and then decoded, with pages given back
    as the windows pass."""
    cfg = CFG_C
    model, w = build(cfg, dtype, seed=8)
    toks = tokens_for(cfg, 400, 7)
    steps, at = [], 0
    for n in [150, 130, 2, 60, 26] + [1] * 32:
        steps.append({"entries": [{"id": "a", "tokens": toks[at:at + n], "want": list(range(n))}], "end": ["a"] if at + n == len(toks) else []})
        at += n
    assert at == len(toks)
    run_and_check(model, steps, cfg, w, {"a": toks}, dtype, "400 tokens", max_tokens=448)


# ---- long decoding, graphs, the entry point ------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_long_decoding_eager_and_from_graphs(dtype):
    cfg = CFG_A
    model, w = build(cfg, dtype, seed=13)
    reqs = {"a": tokens_for(cfg, 150, 1), "b": tokens_for(cfg, 140, 2)}
    steps = [{"entries": [{"id": r, "tokens": t[:6], "want": list(range(6))} for r, t in reqs.items()], "end": []}]
    for i in range(6, 150):
        entries = [{"id": r, "tokens": [t[i]], "want": [0]} for r, t in reqs.items() if i < len(t)]
        steps.append({"entries": entries, "end": [r for r, t in reqs.items() if i == len(t) - 1]})
    run_and_check(model, copy.deepcopy(steps), cfg, w, reqs, dtype, "long decoding", max_tokens=512)
    # a replayed step computes what its eager twin computes, when both split a context's keys for the same longest context
    from tensorline_amd.engine.replay import TraceSession
    plain_session, graph_session = TraceSession(model, 512), TraceSession(model, 512, graphs=True)
    plain_session.runner.fit_context = graph_session.runner.fit_context
    eager = run_steps(model, copy.deepcopy(steps), session=plain_session)
    replayed = run_steps(model, copy.deepcopy(steps), session=graph_session)
    assert graph_session.runner.graph_replays > 100
    for rid, toks in reqs.items():
        for p in range(len(toks)):
            assert rel_error(replayed[rid][p], eager[rid][p]) < 1e-6, f"{rid} at {p}: a graph's step differs from the eager one"


def _greedy(cfg, w, prompts, n):
    want = []
    for p in prompts:
        seq = list(p)
        for _ in range(n):
            seq.append(int(P.forward(w, cfg, seq)[-1].argmax()))
        want.append(seq[len(p):])
    return want


def _folder_weights(folder):
    from safetensors import safe_open
    w = {}
    with safe_open(folder + "/model.safetensors", "pt") as f:
        for k in f.keys():
            w[k] = f.get_tensor(k).float()
    return w


@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_through_the_entry_point(name, tmp_path):
    """``LLM.generate`` with its scheduler, portions under a small token budget, more requests than slots at a
    time, and graphs: in 32-bit the greedy tokens are the plain implementation's."""
    from tensorline_amd import LLM, SamplingParams
    from tensorline_amd.weights.random_init import write_random_model
    cfg = CONFIGS[name]
    folder = write_random_model(typed(cfg), str(tmp_path / "model"), seed=21)
    w = _folder_weights(folder)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (41, 3, 77, 18, 1, 30)]
    want = _greedy(cfg, w, prompts, 12)
    for options in (dict(graphs=False, max_batched_tokens=32, max_num_seqs=3), dict(graphs=True, max_batched_tokens=64, max_num_seqs=4)):
        llm = LLM(folder, dtype="float32", block_size=16 if name == "A" else 8, num_blocks=40 if name == "A" else 80,
                  max_model_len=128, graph_warmup_tokens=0, **options)
        outs = llm.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
        assert [o.token_ids for o in outs] == want
        assert llm.cache.all_free()


def test_command_line_random_model_generate_and_trace_program(tmp_path):
    """The programs a user runs: ``tensorline random-model`` from a config.json, ``tensorline generate`` on the
    folder, and ``bin/trace_run`` fed steps on its standard input."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = copy.deepcopy(CFG_B)
    (tmp_path / "cfg.json").write_text(json.dumps(cfg))
    tl = [sys.executable, os.path.join(root, "bin", "tensorline")]
    folder = str(tmp_path / "m")
    proc = subprocess.run(tl + ["random-model", "--config", str(tmp_path / "cfg.json"), "--out", folder, "--seed", "4"],
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    w = _folder_weights(folder)
    prompts = [tokens_for(cfg, 19, 1), tokens_for(cfg, 4, 2)]
    want = _greedy(cfg, w, prompts, 6)
    base = tl + ["generate", "--model", folder, "--dtype", "float32", "--num-blocks", "32", "--block-size", "8",
                 "--max-tokens", "6", "--stop-token-id", "-1"]
    for p in prompts:
        base += ["--prompt-ids", " ".join(map(str, p))]
    proc = subprocess.run(base, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    recs = [json.loads(l) for l in proc.stdout.splitlines() if l.startswith("{")]
    assert [r["token_ids"] for r in recs] == want
    toks = prompts[0]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": toks[:7], "want": [6]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": toks[7:18], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": toks[18:], "want": [0]}], "end": ["a"]}]
    out = tmp_path / "out"
    proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                           "--max-tokens", "64"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    ref = P.forward(w, cfg, toks).numpy()
    assert not (out / "1.f32").exists()
    for step, place in ((0, 6), (2, 18)):
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(1, -1)
        assert rel_error(got[0], ref[place]) < LIMIT["float32"]


# ---- seeded random configurations ----------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(14))
def test_random_configurations_in_mixed_batches(seed):
    """Sizes, head groupings, layer orders, windows, taps and constants drawn from the seed, a page size of 8, 16 or
    32, five requests cut at random over a pool that holds three: float32 for even seeds, bfloat16 for odd ones."""
    rng = random.Random(2000 + seed)
    cfg = random_config(rng)
    dtype = "float32" if seed % 2 == 0 else "bfloat16"
    model, w = build(cfg, dtype, seed=seed)
    reqs = {f"r{i}": tokens_for(cfg, n, 50 + i) for i, n in enumerate([rng.randint(1, 90) for _ in range(5)])}
    page = rng.choice([8, 16, 32])
    run_and_check(model, mixed_steps(reqs, rng, live=3), cfg, w, reqs, dtype, f"seed {seed}: {cfg}", page_size=page,
                  max_tokens=3 * 96, max_requests=3)
