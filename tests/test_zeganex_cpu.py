"""Zeganex without a GPU: the configuration reader and what it refuses, the spec (schedule, cache and state
needs, tensor names), and pins of the plain implementation (tests/plain_zeganex.py) against closed forms and
against itself in portions."""
import copy
import math

import pytest
import torch

from tensorline_amd.config.model_config import ConfigError
from tensorline_amd.config.registry import get_architecture, known_architectures
from tensorline_amd.models.decoder import DecoderModel
from tensorline_amd.parts.rotary import yarn_frequencies
from tensorline_amd.weights.random_init import random_tensor
from tests import plain_zeganex as P
from tests.zeganex_helpers import CFG_A, CFG_B, CFG_C, YARN, typed


def _model(cfg):
    return DecoderModel(get_architecture("Zeganex").build_spec(typed(cfg)), torch.float32, "cpu")


def _weights(cfg, seed=0, dtype=torch.float64):
    return {n: random_tensor(n, d, seed, "cpu").to(dtype) for n, d in _model(cfg).tensor_decls().items()}


def test_registered_and_round_trips():
    assert "Zeganex" in known_architectures()
    for cfg in (CFG_A, CFG_B, CFG_C):
        t = typed(cfg)
        assert typed(t.to_dict()) == t
    assert typed(CFG_B).bigram is None and typed(CFG_A).bigram == (251, 31, 7)


@pytest.mark.parametrize("edit, text", [
    (lambda c: c["layers"][0].update(type="attention_3"), "unknown"),
    (lambda c: c["layers"][0]["mixer"].pop("conv"), "conv is missing"),
    (lambda c: c["layers"][1]["mixer"].pop("diff"), "diff is missing"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "not a multiple"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=2), "earlier layer"),
    (lambda c: c["layers"][2]["mixer"].update(kv_from=1), "same type"),
    (lambda c: c["layers"][3]["mixer"].update(dim=8), "another dim"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "exceeds"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "unknown"),
    (lambda c: c.pop("norm"), "norm.eps"),
    (lambda c: c["embedding"]["bigram"].update(buckets=0), "positive integer"),
])
def test_reader_refuses(edit, text):
    cfg = copy.deepcopy(CFG_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=text):
        typed(cfg)


def test_spec_schedule_needs_and_names():
    m = _model(CFG_A)
    assert [(e.layer, e.cache_from) for e in m.schedule] == [(0, None), (1, None), (2, 0), (3, 1)]
    needs = m.cache_needs()
    # one key head per map; keys and values share the head size ceil16(max(dim, vdim)); a cache keeps the widest
    # window of its readers, a reader asks for its own
    assert [n.planes[0].shape for n in needs] == [(2, 48), (4, 32), (2, 48), (4, 32)]
    assert [n.window for n in needs] == [21, 47, 13, 47]
    # the last taps - 1 projected rows of q, k, v (of q alone in a layer without keys of its own)
    assert [s.shape[0] for s in m.state_needs()] == [2 * (4 * 24 + 2 * 24 + 2 * 40), 3 * (8 * 16 + 4 * 16 + 2 * 24), 1 * 4 * 24, 2 * 4 * 16]
    assert m.input_state_need().dtype == "int32"
    assert _model(CFG_B).input_state_need() is None and _model(CFG_B).state_needs()[0].shape == (1,)      # one tap keeps nothing
    decls = m.tensor_decls()
    assert decls["bigram"].shape == (252, 96) and decls["l0.mix.q.conv"].shape == (96, 3) and decls["l1.mix.k"].shape == (64, 96)
    assert "l2.mix.k" not in decls and "l2.norm2" not in decls and "l2.mix.g" in decls and "l0.mix.o.b" in decls
    assert "l1.mlp.e5.up" in decls and "l1.mlp.e0.gate" not in decls and "l1.mix.lq2" in decls and "l1.mix.o.b" not in decls
    from tensorline_amd.cache.manager import CacheManager
    cache = CacheManager(needs, m.schedule, m.state_needs(), page_size=16, num_blocks=8, max_requests=2, dtype=torch.float32,
                         device="cpu", input_state_need=m.input_state_need())
    assert len(cache.groups) == 2 and cache.storage(2)["k"] is cache.storage(0)["k"] and not cache.owns_storage(3)
    assert cache.state["input"].dtype == torch.int32 and not cache.prefix_caching


def test_yarn_table_of_the_framework_is_the_plain_one():
    for dims, base, scaling in ((8, 500.0, YARN), (20, 50.0, None), (32, 10000.0, {"factor": 3.0, "original": 512, "fast": 24.0, "slow": 1.5}),
                                (2, 7.0, {"factor": 1.5, "original": 16, "fast": 4.0, "slow": 1.0})):
        f, mag = yarn_frequencies(dims, base, scaling)
        pf, pmag = P.yarn_table(dims, base, scaling)
        assert torch.allclose(f.double(), pf, rtol=1e-6) and abs(mag - pmag) < 1e-12
    f, mag = P.yarn_table(16, 100.0, {"factor": 8.0, "original": 32, "fast": 8.0, "slow": 1.0})
    assert abs(mag - (0.1 * math.log(8.0) + 1.0)) < 1e-12
    plain = torch.tensor([100.0 ** (-2.0 * i / 16) for i in range(8)], dtype=torch.float64)
    assert torch.allclose(f[0], plain[0]) and torch.allclose(f[-1], plain[-1] / 8.0)          # fast pairs kept, slow ones stretched


def test_rotation_turns_neighbours_and_leaves_the_rest():
    x = torch.randn(5, 2, 12, dtype=torch.float64)
    pos = torch.tensor([0, 1, 7, 100, 1000])
    y = P.rotate_pairs(x, pos, {"dims": 4, "base": 10.0, "scaling": None})
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.allclose(y[0], x[0])
    a = 7 * 10.0 ** (-2.0 * 1 / 4)
    assert torch.allclose(y[2, 1, 2], x[2, 1, 2] * math.cos(a) - x[2, 1, 3] * math.sin(a))
    assert torch.allclose(y[2, 1, 3], x[2, 1, 3] * math.cos(a) + x[2, 1, 2] * math.sin(a))
    # a score between rotated queries and keys depends on the distance alone
    q, k = torch.randn(1, 1, 4, dtype=torch.float64), torch.randn(1, 1, 4, dtype=torch.float64)
    rot = {"dims": 4, "base": 10.0, "scaling": None}
    s = lambda i, j: (P.rotate_pairs(q, torch.tensor([i]), rot) * P.rotate_pairs(k, torch.tensor([j]), rot)).sum()
    assert torch.allclose(s(9, 4), s(105, 100))


def test_bigram_rows():
    assert P.bigram_rows([5, 6, 7], None, 13, 3, 2) == [13, (5 * 3 + 6 * 2) % 13, (6 * 3 + 7 * 2) % 13]
    assert P.bigram_rows([6, 7], 5, 13, 3, 2) == P.bigram_rows([5, 6, 7], None, 13, 3, 2)[1:]


def test_window_counts_itself():
    q = torch.zeros(6, 3, dtype=torch.float64)
    v = torch.eye(6, dtype=torch.float64)
    pos = torch.arange(6)
    out = P.windowed_softmax_attention(q, q, v, 1.0, pos, pos, 3)
    assert torch.allclose(out[5], torch.tensor([0, 0, 0, 1 / 3, 1 / 3, 1 / 3], dtype=torch.float64))
    assert torch.allclose(out[1], torch.tensor([0.5, 0.5, 0, 0, 0, 0], dtype=torch.float64))
    assert torch.allclose(P.windowed_softmax_attention(q, q, v, 1.0, pos, pos, 0)[5], torch.full((6,), 1 / 6, dtype=torch.float64))


def test_router_keeps_the_softmax_over_all():
    w = {"r.router": torch.tensor([[1.0], [3.0], [2.0], [0.0]], dtype=torch.float64)}
    chosen, weights = P.router_choice(torch.ones(1, 1, dtype=torch.float64), w, "r.", 2)
    e = torch.exp(torch.tensor([1.0, 3.0, 2.0, 0.0], dtype=torch.float64))
    assert chosen.tolist() == [[1, 2]] and torch.allclose(weights[0], (e / e.sum())[[1, 2]]) and weights.sum() < 1.0


def test_two_maps_with_equal_queries_cancel_to_the_factor():
    """Both maps alike (the same rows for map 1 and map 2): o = (1 - lambda) a, which the norm per head takes away
    but for the sign; the output is rms_divide(a) * (1 - diff) * sign(1 - lambda)."""
    cfg = copy.deepcopy(CFG_A)
    w = _weights(cfg, 3)
    p, m = "l1.mix.", cfg["layers"][1]["mixer"]
    for name, heads in (("q", m["heads"]), ("k", m["kv_heads"])):
        for suffix in ("", ".b", ".conv"):
            t = w[p + name + suffix].view(heads, 2, m["dim"], *w[p + name + suffix].shape[1:])
            t[:, 1] = t[:, 0]
    h = torch.randn(9, cfg["width"], dtype=torch.float64)
    pos = torch.arange(9)
    lam = P.differential_lambda(w, p, m["diff"])
    out = P.differential_attention(h, w, p, m, pos, 1e-5, P.MixerMemory())
    # the same through one map of a plain softmax attention
    T, H, G, d, dv = 9, m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = P.short_conv(h @ w[p + "q"].T + w[p + "q.b"], w[p + "q.conv"])[0].view(T, H, 2, d)[:, :, 0]
    k = P.short_conv(h @ w[p + "k"].T + w[p + "k.b"], w[p + "k.conv"])[0].view(T, G, 2, d)[:, :, 0]
    v = P.short_conv(h @ w[p + "v"].T + w[p + "v.b"], w[p + "v.conv"])[0].view(T, G, dv)
    a = torch.stack([P.windowed_softmax_attention(q[:, i], k[:, i // (H // G)], v[:, i // (H // G)], m["scale"], pos, pos, 33)
                     for i in range(H)], dim=1)
    want = (P.rms_divide((1.0 - lam) * a, 1e-5) * (1.0 - m["diff"])).reshape(T, H * dv) @ w[p + "o"].T
    assert torch.allclose(out, want, atol=1e-9)


@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_plain_in_portions_and_token_by_token_equals_whole(name):
    cfg = {"A": CFG_A, "B": CFG_B, "C": CFG_C}[name]
    w = _weights(cfg, 5)
    g = torch.Generator().manual_seed(1)
    toks = torch.randint(0, cfg["vocab"], (70,), generator=g).tolist()
    whole = P.forward(w, cfg, toks)
    for sizes in ((1,), (2, 1, 17, 3), (64, 6)):
        mem, rows, at, k = P.SequenceMemory(cfg), [], 0, 0
        while at < len(toks):
            n = min(sizes[k % len(sizes)], len(toks) - at)
            rows.append(P.forward(w, cfg, toks[at:at + n], mem))
            at, k = at + n, k + 1
        assert torch.allclose(torch.cat(rows), whole, atol=1e-9), sizes


def test_a_key_outside_the_window_changes_nothing_in_one_layer():
    """One layer, window 5, two taps: the output at position i depends on inputs i - 5 .. i only (the window's oldest
    key carries one more input through its convolution)."""
    from tests.zeganex_helpers import _rotary, one_layer
    cfg = one_layer("attention_2", _rotary(2, 1, 8, 8, 2, 5, 4), width=16)
    w = _weights(cfg, 2)
    h = torch.randn(12, 16, dtype=torch.float64)
    pos = torch.arange(12)
    run = lambda x: P.gated_rotary_attention(x, w, "l0.mix.", cfg["layers"][0]["mixer"], pos, P.MixerMemory())
    base = run(h)
    h2 = h.clone()
    h2[5] += 3.0                         # position 11 sees keys 7 .. 11, built from inputs 6 .. 11
    assert torch.allclose(run(h2)[11], base[11]) and not torch.allclose(run(h2)[10], base[10])
