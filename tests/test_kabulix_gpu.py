"""Kabulix on the GPU against the plain implementation (tests/plain_kabulix.py): every mechanism alone, whole
prompts, token-by-token decoding, portions, mixed batches with pages and slots used again, tokens made to stand out
at the places where a cache, a window or a chunk can lose them, long decoding, and greedy generation through the
entry point."""
import copy
import random

import numpy as np
import pytest
import torch

from tests import plain_kabulix as P
from tests.helpers import steps_portions, steps_prefill_then_decode, steps_whole
from tests.kabulix_helpers import (CFG_A, CFG_B, CFG_C, CONFIGS, YARN, _chunked, _dense, _latent, _moe, _windowed, build,
                                   one_layer, random_config, routed_layers, typed)
from tests.samovik_helpers import rel_error, run_steps
from tests.test_samovik_gpu import mixed_steps
from tests.tumitar_helpers import run_steps_with_routes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]
LIMIT = {"float32": 2e-5, "bfloat16": 5e-2}          # of the logits' own root mean square


def tokens_for(cfg, n, seed):
    rng = random.Random(seed)
    return [rng.randrange(cfg["vocab"]) for _ in range(n)]


def run_and_check(model, steps, cfg, w, reqs, dtype, what="", **kw):
    """Run the steps and hold every position against the plain implementation.  In float32 the plain run routes by
    itself.  In bfloat16 a router's close call may fall the other way and then changes every later position through
    the caches: there the plain run is told which experts the framework chose, and every such choice must be what
    the plain router chooses once its logits may move by a tenth of their spread."""
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
        seen = {}
        want = P.forward(cfg, w, toks, forced_experts=forced, router_logits=seen).numpy()
        for layer, taken in (forced or {}).items():
            z = seen[layer]
            for t in range(len(toks)):
                slack = 0.1 * max(float(z[t].std()) if z.shape[1] > 1 else 1.0, 0.05)
                assert P.is_close_call(z[t], taken[t], cfg["layers"][layer]["mlp"], slack), \
                    f"{what}: request {rid}, layer {layer}, position {t}: the experts {taken[t].tolist()} are not the router's choice"
        rows = got[rid]
        assert sorted(rows) == list(range(len(toks))), f"{what}: {rid} is missing positions"
        errs = {p: rel_error(rows[p], want[p]) for p in rows}
        first_bad = next((p for p in sorted(rows) if not errs[p] <= LIMIT[dtype]), None)
        assert first_bad is None, (f"{what} {dtype}: request {rid}: first wrong position {first_bad} of {len(toks)}, "
                                   f"worst error {max(errs.values()):.3e}")


def _session(model, page=16, blocks=64, slots=4):
    from tensorline_amd.cache.manager import CacheManager
    from tensorline_amd.engine.runner import ModelRunner
    cache = CacheManager(model.cache_needs(), model.schedule, model.state_needs(), page_size=page, num_blocks=blocks,
                         max_requests=slots, dtype=model.dtype, device=DEV, input_state_need=model.input_state_need())
    return cache, ModelRunner(model, cache)


def _step_context(cache, runner, portions):
    """``portions``: (request, first position, count).  Returns the step's context and cache views."""
    from tensorline_amd.engine.batch import StepEntry
    entries = []
    for rid, lo, n in portions:
        if not cache.has_request(rid):
            cache.add_request(rid)
        cache.grow(rid, lo + n)
        entries.append(StepEntry(rid, [0] * n, lo, [0]))
    packed = runner.pack(entries)
    return runner.context(packed, runner._upload(packed.data))


def _rms_error(got, want):
    return ((got - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()).item()


# ---- every mechanism alone -------------------------------------------------------------------------
@pytest.mark.parametrize("case", [
    # query heads, key heads, dim, vdim, turned dims, normed, values are the keys
    (4, 2, 24, 24, 8, True, True), (8, 4, 16, 40, 0, False, False), (3, 1, 10, 7, 10, True, False), (2, 2, 128, 128, 32, True, True),
    (1, 1, 6, 6, 2, False, True), (5, 5, 250, 250, 250, True, True), (6, 2, 64, 32, 64, True, False)])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_head_norm_rotation_and_cache_write_in_one_pass(case, dtype):
    from tensorline_amd.ops import kernels
    from tensorline_amd.parts.rotary import yarn_frequencies
    H, G, d, dv, rot, normed, from_keys = case
    D = -(-max(d, dv) // 16) * 16
    T, page, pages = 23, 8, 9
    torch.manual_seed(sum(case[:5]))
    cols = (H + G) * d + (0 if from_keys else G * dv)
    proj = torch.randn(T, cols + 5)
    pos = torch.randint(0, 100, (T,), dtype=torch.int32)
    slots = torch.randperm(pages * page)[:T].to(torch.int32)
    wq, wk = torch.randn(d) + 1, torch.randn(d) + 1
    freq, mag = yarn_frequencies(rot, 300.0, YARN) if rot else (None, 1.0)
    kc = torch.full((pages, page, G, D), 7.0).to(dtype).to(DEV)
    vc = torch.full((pages, G, D, page), 7.0).to(dtype).to(DEV)
    got_q = kernels.head_norm_rotate_store(proj.to(DEV), pos.to(DEV), wq.to(DEV) if normed else None, wk.to(DEV) if normed else None,
                                           1e-5, freq.to(DEV) if rot else None, mag, kc, vc, slots.to(DEV), H, G, d, dv, from_keys, dtype)
    x = proj.double()
    q, k = x[:, :H * d].view(T, H, d), x[:, H * d:(H + G) * d].view(T, G, d)
    v = k.clone() if from_keys else x[:, (H + G) * d:(H + G) * d + G * dv].view(T, G, dv)
    if normed:
        q, k = P.norm_plain(q, wq.double(), 1e-5), P.norm_plain(k, wk.double(), 1e-5)
    if rot:
        freqs, m = P.frequencies(rot, 300.0, YARN)
        q, k = P.turn_pairs(q, pos.tolist(), freqs, m), P.turn_pairs(k, pos.tolist(), freqs, m)
    # angles are float32 products of positions up to 100: 6e-6 of a radian, on values of up to six or so
    tol = dict(atol=2e-4, rtol=1e-4) if dtype == torch.float32 else dict(atol=3e-2, rtol=2e-2)
    got_q = got_q.double().cpu().view(T, H, D)
    torch.testing.assert_close(got_q[:, :, :d], q, **tol)
    assert not got_q[:, :, d:].any()
    got_k = kc.double().cpu().view(-1, G, D)[slots.long()]
    torch.testing.assert_close(got_k[:, :, :d], k, **tol)
    assert not got_k[:, :, d:].any()
    got_v = vc.double().cpu().permute(0, 3, 1, 2).reshape(-1, G, D)[slots.long()]
    torch.testing.assert_close(got_v[:, :, :v.shape[2]], v, **tol)
    assert not got_v[:, :, v.shape[2]:].any()
    untouched = torch.ones(pages * page, dtype=torch.bool)
    untouched[slots.long()] = False
    assert (kc.float().cpu().view(-1, G, D)[untouched] == 7.0).all()


@pytest.mark.parametrize("experts,groups,keep,top", [(15, 3, 2, 5), (8, 8, 3, 3), (6, 1, 1, 6), (128, 8, 2, 9), (200, 4, 1, 32),
                                                      (4, 2, 2, 1), (64, 64, 64, 5), (9, 3, 1, 3)])
def test_router_chooses_within_the_best_groups(experts, groups, keep, top):
    from tensorline_amd.ops import kernels
    torch.manual_seed(experts + groups)
    z = (torch.randn(40, experts + 3) * 2).float()
    z[1, :experts] = 0.25                                 # all equal: lower groups and lower indices win
    z[2, :experts] = torch.arange(experts).float() % 2    # many ties
    ids, wts = kernels.moe_route(z.to(DEV), top, "sigmoid_grouped", experts=experts, groups=groups, keep=keep)
    for t in range(z.shape[0]):
        chosen, weights = P.route(z[t, :experts].double(), top, groups, keep)
        assert ids[t].tolist() == chosen, f"row {t}"
        assert torch.allclose(wts[t].cpu().double(), torch.tensor(weights, dtype=torch.float64), atol=1e-6)
    assert torch.allclose(wts.sum(1).cpu(), torch.ones(z.shape[0]), atol=1e-5)


def test_groups_keep_a_larger_score_out():
    """The largest score of all lies in a group whose two best sum to less than another group's: it is not chosen."""
    from tensorline_amd.ops import kernels
    z = torch.tensor([[4.0, -9.0, -9.0, 1.5, 1.4, 1.3]])
    ids, _ = kernels.moe_route(z.to(DEV), 2, "sigmoid_grouped", groups=2, keep=1)
    assert ids.tolist() == [[3, 4]]
    assert P.route(z[0].double(), 2, 2, 1)[0] == [3, 4]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gated_activations(dtype):
    from tensorline_amd.ops import kernels
    torch.manual_seed(1)
    gu = (torch.randn(9, 2 * 37) * 3)
    for name, act in (("gelu_tanh", P.gelu_tanh), ("silu", P.silu)):
        got = kernels.glu(gu.to(DEV), name, dtype).double().cpu()
        want = act(gu[:, :37].double()) * gu[:, 37:].double()
        torch.testing.assert_close(got, want, atol=1e-5 if dtype == torch.float32 else 5e-2, rtol=1e-5 if dtype == torch.float32 else 1e-2)


MIXERS = [
    ("attention", _windowed(4, 2, 24, 21, 3, 8)),
    ("attention", _windowed(1, 1, 10, 3, 0, 10, base=20.0)),                        # small and odd, full rotation, nothing kept
    ("attention", _windowed(6, 1, 64, 40, 20, 32, scaling=YARN)),                   # matrix-core attention, more kept than a page
    ("attention", _windowed(2, 2, 128, 500, 4, 0, scale=0.03)),                     # no rotation, a window wider than the sequence
    ("attention", _windowed(18, 2, 32, 100, 1, 2)),                                 # nine query heads a group
    ("attention", _windowed(4, 4, 48, 16, 16, 48)),                                 # the window and the kept tokens one page each
    ("latent_attention", _latent(3, 16, 8, 24, 40, 13)),
    ("latent_attention", _latent(1, 6, 2, 9, 11, 1, scaling=None)),                 # a window of the token itself
    ("latent_attention", _latent(4, 32, 16, 32, 48, 0)),                            # no window
    ("latent_attention", _latent(2, 24, 32, 16, 96, 70, base=50.0)),                # a cached row of 128
    ("latent_attention", _latent(2, 16, 8, 8, 300, 33)),                            # a cached row wider than the matrix-core kernels take
    ("attention_2", _chunked(4, 2, 24, 40, 19)),
    ("attention_2", _chunked(3, 1, 10, 7, 16, scale=0.4)),
    ("attention_2", _chunked(2, 2, 128, 96, 0, scale=0.05)),                        # no chunk
    ("attention_2", _chunked(4, 1, 32, 32, 48)),                                    # matrix-core attention
    ("attention_2", _chunked(9, 3, 64, 16, 1, scale=0.1)),                          # a chunk of one token
    ("attention_2", _chunked(2, 1, 64, 64, 200)),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(MIXERS)))
def test_mixer_alone(case, dtype):
    """Three sequences in one batch, each from its first token, then each continued by a second step of other
    sizes (one token among them): the mixer's outputs against the plain ones of the whole sequences."""
    kind, mixer = MIXERS[case]
    cfg = one_layer(kind, mixer, width=72)
    model, w = build(cfg, dtype, seed=case)
    W = P.as_double(w)
    first, second = [37, 1, 150], [1, 20, 3]
    torch.manual_seed(case)
    hs = [torch.randn(a + b, 72).to(torch.bfloat16).float() for a, b in zip(first, second)]
    cache, runner = _session(model)
    mix = model.blocks[0].mixer
    ctx, views = _step_context(cache, runner, [(i, 0, n) for i, n in enumerate(first)])
    got1 = mix.forward(torch.cat([h[:n] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    for i, n in enumerate(first):
        cache.trim(i, n)
    ctx, views = _step_context(cache, runner, [(i, a, b) for i, (a, b) in enumerate(zip(first, second))])
    got2 = mix.forward(torch.cat([h[n:] for h, n in zip(hs, first)]).to(DEV).to(model.dtype), ctx, views[0]).float().cpu()
    at1 = at2 = 0
    for h, a, b in zip(hs, first, second):
        want = P.mixer(kind, h.double(), list(range(a + b)), W, "l0.mix.", mixer, 1e-6).float()
        got = torch.cat((got1[at1:at1 + a], got2[at2:at2 + b]))
        err = _rms_error(got, want)
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{kind} {mixer}: sequence of {a} + {b}: {err:.3e}"
        at1, at2 = at1 + a, at2 + b


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("mlp", [_dense(136), _dense(7), _moe(6, 2, 40, groups=3, keep=2, shared=24), _moe(3, 3, 20), _moe(1, 1, 100, shared=5),
                                 _moe(40, 5, 16, groups=8, keep=3), _moe(4, 2, 24, groups=4, keep=2)])
def test_feed_forward_alone(mlp, dtype):
    """Few rows and many (the grouped product's tiles of 16 and of 64 rows)."""
    cfg = one_layer("attention_2", _chunked(1, 1, 8, 8, 4), mlp, width=88)
    model, w = build(cfg, dtype, seed=3)
    W = P.as_double(w)
    ff = model.blocks[0].feed_forward
    for rows in (1, 5, 300):
        torch.manual_seed(rows)
        h = (torch.randn(rows, 88) * 2).to(torch.bfloat16).float()
        got = ff.forward(h.to(DEV).to(model.dtype), None).float().cpu()
        want = (P.gated_ff(h.double(), W, "l0.mlp.", P.gelu_tanh) if mlp["kind"] == "dense" else P.ff_experts(h.double(), W, "l0.mlp.", mlp)).float()
        err = (got - want).abs().max().item() / want.abs().max().item()
        assert err < (1e-5 if dtype == "float32" else 3e-2), f"{rows} rows: {err:.3e}"


def test_norm_weights_are_stored_around_zero():
    cfg = one_layer("attention_2", _chunked(1, 1, 8, 8, 4), None, width=40)
    model, w = build(cfg, "float32", seed=5)
    x = torch.randn(6, 40)
    got = model.blocks[0].mixer_norm.forward(x.to(DEV).clone(), None).cpu()
    assert torch.allclose(got, P.norm_around_zero(x.double(), w["l0.norm1"].double(), 1e-6).float(), atol=1e-5)
    assert abs(float(w["l0.norm1"].mean())) < 0.2            # the random weights lie around zero, as a checkpoint's do


# ---- a token made loud: what a wrong window, chunk, kept token or a lost page would show ----------------------
LOUD = [
    ("attention", _windowed(4, 2, 64, 37, 5, 16, scale=0.2), (0, 4, 5, 15, 16, 31, 230)),
    ("attention", _windowed(2, 1, 32, 48, 18, 32, scale=0.3), (0, 16, 17, 18, 47, 48, 100)),
    ("latent_attention", _latent(4, 32, 16, 32, 48, 37, scale=0.2), (0, 15, 16, 31, 230)),
    ("attention_2", _chunked(4, 2, 64, 64, 50, scale=0.2), (0, 49, 50, 99, 100, 249)),
    ("attention_2", _chunked(2, 2, 32, 48, 48, scale=0.3), (15, 16, 47, 48, 143, 144)),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("case", range(len(LOUD)))
def test_a_loud_token_at_the_edges_of_windows_chunks_and_pages(case, dtype):
    """One input row of the mixer is made twenty-five times as large as the others, so that what it leaves in the
    cache dominates whatever reads it: whether it is seen shows in every output around it.  It sits at the
    sequence's first token, among the kept first tokens and right behind them, at both sides of a page's border,
    of a window's and a chunk's edge, and hundreds of tokens back; the outputs are computed as one prompt, as
    portions cut at the edge where it drops out of sight, and decoded one by one across that edge, with pages given
    back as the layer allows."""
    kind, mixer, places = LOUD[case]
    cfg = one_layer(kind, mixer, width=64)
    model, w = build(cfg, dtype, seed=9)
    W = P.as_double(w)
    mix = model.blocks[0].mixer
    n = 300
    mask = mixer["mask"]
    for loud in places:
        torch.manual_seed(loud)
        h = torch.randn(n, 64)
        h[loud] *= 25.0
        h = h.to(torch.bfloat16).float()
        want = P.mixer(kind, h.double(), list(range(n)), W, "l0.mix.", mixer, 1e-6).float()
        if kind == "attention_2":
            edge = (loud // mask["size"] + 1) * mask["size"]            # the first position that does not see it
        else:
            edge = loud + mask["size"] if loud >= mask.get("keep_first", 0) else n
        edge = min(edge, n - 2)
        cuts = {"whole": [n], "cut at the edge": [edge, 2, n], "decoded across the edge": [max(edge - 3, 1)] + [1] * 8 + [n],
                "portions of two": [max(edge - 5, 1)] + [2] * 5 + [n]}
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
                err = _rms_error(got[lo:hi], want[lo:hi])
                assert err < tol, f"{kind} {mask}, loud token at {loud}, {name}: positions {lo}..{hi}: {err:.3e}"
    # the loud token does show where it is seen, and only there (in the plain outputs that everything is held against)
    h = torch.randn(n, 64, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16).double()
    loud = places[-2]
    quiet = P.mixer(kind, h, list(range(n)), W, "l0.mix.", mixer, 1e-6)
    h2 = h.clone()
    h2[loud] *= 25.0
    shown = (P.mixer(kind, h2, list(range(n)), W, "l0.mix.", mixer, 1e-6) - quiet).abs().amax(1)
    edge = (loud // mask["size"] + 1) * mask["size"] if kind == "attention_2" else loud + mask["size"]
    assert float(shown[loud:min(edge, n)].min()) > 1e-5 and (edge >= n or float(shown[edge:].max()) == 0.0)


def test_pages_behind_a_window_go_back_and_kept_first_pages_stay():
    cfg = one_layer("attention", _windowed(2, 1, 16, 20, 18, 8), None, width=32)
    model, _ = build(cfg, "float32", seed=1)
    cache, runner = _session(model, blocks=12)
    cache.add_request("a")
    assert cache.grow("a", 100)
    cache.trim("a", 100)
    table = cache.table_array("a", 0).tolist()
    assert all(p >= 0 for p in table[:2]) and all(p < 0 for p in table[2:5]) and all(p >= 0 for p in table[5:7])
    cfg = one_layer("attention_2", _chunked(2, 1, 16, 16, 40), None, width=32)
    model, _ = build(cfg, "float32", seed=1)
    cache, runner = _session(model, blocks=12)
    cache.add_request("a")
    assert cache.grow("a", 100)
    cache.trim("a", 100)                      # the token at position 100 sees its chunk from position 80 on
    table = cache.table_array("a", 0).tolist()
    assert all(p < 0 for p in table[:5]) and all(p >= 0 for p in table[5:7])
    # a request far longer than the pool runs through it, because pages come back
    assert cache.can_ever_hold(5000, 64) and not cache.can_ever_hold(5000, 200)


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
    """A request of one token, then one of two, then one decoded from its first token on, all through one slot and
    the same few pages: nothing of an earlier request reaches the next."""
    cfg = CFG_A
    model, w = build(cfg, "float32", seed=6)
    reqs = {"p": tokens_for(cfg, 1, 1), "q": tokens_for(cfg, 2, 2), "r": tokens_for(cfg, 40, 3), "s": tokens_for(cfg, 5, 4)}
    steps = steps_whole({"p": reqs["p"], "q": reqs["q"]}) + steps_portions({"r": reqs["r"]}, sizes=(1,)) + steps_whole({"s": reqs["s"]})
    run_and_check(model, steps, cfg, w, reqs, "float32", "first tokens", max_tokens=64, max_requests=1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_long_request_through_a_small_pool(dtype):
    """400 tokens in portions and then decoded, through windows, kept first tokens and chunks, with pages given back
    as they pass; the kept first tokens are read hundreds of positions later."""
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
            seq.append(int(P.forward(cfg, w, seq)[-1].argmax()))
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
    ref = P.forward(cfg, w, toks).numpy()
    assert not (out / "1.f32").exists()
    for step, place in ((0, 6), (2, 18)):
        got = np.fromfile(out / f"{step}.f32", dtype="<f4").reshape(1, -1)
        assert rel_error(got[0], ref[place]) < LIMIT["float32"]


# ---- seeded random configurations ----------------------------------------------------------------------------
@pytest.mark.parametrize("seed", range(14))
def test_random_configurations_in_mixed_batches(seed):
    """Sizes, head groupings, layer orders, windows, kept tokens, chunks and constants drawn from the seed, a page size
    of 8, 16 or 32, five requests cut at random over a pool that holds three: float32 for even seeds, bfloat16 for
    odd ones."""
    rng = random.Random(3000 + seed)
    cfg = random_config(rng)
    dtype = "float32" if seed % 2 == 0 else "bfloat16"
    model, w = build(cfg, dtype, seed=seed)
    reqs = {f"r{i}": tokens_for(cfg, n, 50 + i) for i, n in enumerate([rng.randint(1, 90) for _ in range(5)])}
    page = rng.choice([8, 16, 32])
    run_and_check(model, mixed_steps(reqs, rng, live=3), cfg, w, reqs, dtype, f"seed {seed}: {cfg}", page_size=page,
                  max_tokens=3 * 96, max_requests=3)
