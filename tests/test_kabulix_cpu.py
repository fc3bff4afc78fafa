"""Kabulix without a GPU: the configuration reader and what it refuses, the spec (mixer kinds, cache needs, tensor
names), what the cache manager gives back behind windows and chunks, and pins of the plain implementation
(tests/plain_kabulix.py) against closed forms."""
import copy
import math

import pytest
import torch

from tensorline_amd.cache.manager import CacheManager
from tensorline_amd.config.model_config import ConfigError
from tensorline_amd.config.registry import get_architecture, known_architectures
from tensorline_amd.models.decoder import DecoderModel
from tensorline_amd.parts.rotary import yarn_frequencies
from tensorline_amd.parts.spec import keys_and_values
from tensorline_amd.weights.random_init import random_tensor
from tests import plain_kabulix as P
from tests.kabulix_helpers import CFG_A, CFG_B, CFG_C, YARN, _chunked, _latent, _moe, _windowed, one_layer, typed


def _model(cfg):
    return DecoderModel(get_architecture("Kabulix").build_spec(typed(cfg)), torch.float32, "cpu")


def _weights(cfg, seed=0):
    return {n: random_tensor(n, d, seed, "cpu").to(torch.float64) for n, d in _model(cfg).tensor_decls().items()}


def test_registered_and_round_trips():
    assert "Kabulix" in known_architectures()
    for cfg in (CFG_A, CFG_B, CFG_C):
        t = typed(cfg)
        assert typed(t.to_dict()) == t


@pytest.mark.parametrize("edit, text", [
    (lambda c: c["layers"][0].update(type="attention_3"), "unknown"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale is missing"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank is missing"),
    (lambda c: c["layers"][0]["mixer"].update(heads=3), "not a multiple"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim equals dim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot_dim"),
    (lambda c: c["layers"][2]["mixer"].update(rot={"dims": 2, "base": 10.0}), "no rotation"),
    (lambda c: c["layers"][2]["mixer"]["mask"].update(keep_first=2), "keep_first"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "exceeds"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "equal groups"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "unknown"),
    (lambda c: c.pop("norm"), "norm.eps"),
])
def test_reader_refuses(edit, text):
    cfg = copy.deepcopy(CFG_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=text):
        typed(cfg)


def test_spec_kinds_needs_and_names():
    m = _model(CFG_A)
    kinds = [type(b.mixer).__name__ for b in m.blocks]
    assert kinds == ["MaskedAttention", "LatentAttention", "MaskedAttention", "MaskedAttention"]
    needs = m.cache_needs()
    assert [(n.window, n.keep_first, n.chunk) for n in needs] == [(21, 3, 0), (13, 0, 0), (0, 0, 19), (33, 17, 0)]
    # keys and values share the head size ceil16(max(dim, vdim)); the latent layer caches one row for all heads
    assert [n.planes[0].shape for n in needs] == [(2, 32), (1, 64), (2, 48), (2, 16)]
    assert all(n is None for n in m.state_needs())
    names = set(m.tensor_decls())
    assert {"embed", "final.norm", "l0.mix.q.b", "l0.mix.k.b", "l0.mix.q.norm", "l0.mix.k.norm", "l1.mix.dkv.norm", "l1.mix.uk",
            "l1.mix.g", "l2.mix.g", "l2.mix.v", "l1.mlp.router", "l1.mlp.shared.sg", "l1.mlp.e5.gate", "l3.mlp.e7.down"} <= names
    assert not {"l0.mix.v", "l0.mix.g", "l2.mix.q.b", "l2.norm2", "l3.mlp.shared.sg", "head"} & names
    decls = m.tensor_decls()
    assert decls["l0.mix.q.norm"].shape == (24,) and decls["l1.mix.g"].shape == (3 * 24, 96) and decls["l2.mix.g"].shape == (4, 96)
    assert decls["l1.mlp.shared.sg"].shape == (1, 96)
    assert m.blocks[2].feed_forward is None


def test_cache_manager_gives_pages_back_behind_windows_and_chunks_but_keeps_the_first():
    from tensorline_amd.parts.spec import ScheduleEntry
    needs = [keys_and_values(1, 16, window=20, keep_first=18), keys_and_values(1, 16, chunk=40), keys_and_values(1, 16)]
    cache = CacheManager(needs, [ScheduleEntry(i) for i in range(3)], [None] * 3, page_size=16, num_blocks=12, max_requests=2,
                         dtype=torch.float32, device="cpu", allocate_storage=False)
    assert len(cache.groups) == 3 and cache.has_windows
    cache.add_request("a")
    assert cache.grow("a", 100)
    assert cache.trim("a", 100) == 3 + 5
    held = lambda g: [p >= 0 for p in cache.table_array("a", g).tolist()]
    assert held(0) == [True, True, False, False, False, True, True]        # positions 0..17 kept, 81.. in the window
    assert held(1) == [False] * 5 + [True, True]                            # position 100's chunk starts at 80
    assert all(held(2))
    assert cache.trim("a", 100) == 0
    assert cache.grow("a", 130) and cache.trim("a", 130) == 1 + 2
    assert held(0)[:2] == [True, True]
    cache.release("a")
    assert cache.all_free()


def test_mask_parameter_of_the_mixer():
    from tensorline_amd.parts.masked_attention import read_mask
    assert read_mask("x", None) == (0, 0, 0)
    assert read_mask("x", {"kind": "window", "size": 9, "keep_first": 2}) == (9, 2, 0)
    assert read_mask("x", {"kind": "chunk", "size": 5}) == (0, 0, 5)
    for bad in ({"kind": "chunk", "size": 5, "keep_first": 1}, {"kind": "window", "size": 0}, {"kind": "stripes", "size": 4}):
        with pytest.raises(ValueError):
            read_mask("x", bad)


# ---- pins of the plain implementation ---------------------------------------------------------------------
def test_yarn_table_of_the_framework_is_the_plain_one():
    for dims, base, scaling in ((8, 500.0, YARN), (32, 50000.0, {"factor": 8.0, "original": 512, "fast": 32.0, "slow": 1.0}),
                                (20, 50.0, None), (2, 10.0, YARN)):
        f, mag = yarn_frequencies(dims, base, scaling)
        want, want_mag = P.frequencies(dims, base, scaling)
        assert torch.allclose(f.double(), torch.tensor(want, dtype=torch.float64), rtol=1e-6) and abs(mag - want_mag) < 1e-12
    f, mag = P.frequencies(8, 100.0, None)
    assert f == [1.0, 100.0 ** -0.25, 0.1, 100.0 ** -0.75] and mag == 1.0


def test_rotation_turns_neighbours_and_leaves_the_rest():
    x = torch.arange(1.0, 7.0, dtype=torch.float64).view(1, 6)
    got = P.turn_pairs(x.repeat(2, 1), [0, 3], [0.5, 2.0], 1.0)
    assert torch.equal(got[0], x[0])                                         # position 0 turns nothing
    a, b = 1.5, 6.0
    want = torch.tensor([1 * math.cos(a) - 2 * math.sin(a), 2 * math.cos(a) + 1 * math.sin(a),
                         3 * math.cos(b) - 4 * math.sin(b), 4 * math.cos(b) + 3 * math.sin(b), 5.0, 6.0], dtype=torch.float64)
    assert torch.allclose(got[1], want)
    assert torch.allclose((got[1, :4] ** 2).sum(), (x[0, :4] ** 2).sum())    # lengths stay


def test_who_sees_whom():
    assert [j for j in range(12) if P.sees_window_and_first(11, j, 4, 2)] == [0, 1, 8, 9, 10, 11]
    assert [j for j in range(12) if P.sees_window_and_first(3, j, 4, 2)] == [0, 1, 2, 3]
    assert [j for j in range(12) if P.sees_window(11, j, 4)] == [8, 9, 10, 11]
    assert [j for j in range(12) if P.sees_window(5, j, 1)] == [5]
    assert [j for j in range(12) if P.sees_chunk(9, j, 4)] == [8, 9]
    assert [j for j in range(12) if P.sees_chunk(8, j, 4)] == [8]
    assert [j for j in range(12) if P.sees_chunk(7, j, 4)] == [4, 5, 6, 7]


def test_router_groups_and_weights():
    z = torch.tensor([4.0, -9.0, -9.0, 1.5, 1.4, 1.3], dtype=torch.float64)
    # the first group holds the largest score, but its two best sum to less than the second group's
    assert P.route(z, 2, 2, 1)[0] == [3, 4]
    chosen, weights = P.route(z, 2, 2, 2)
    assert chosen == [0, 3]
    s = torch.sigmoid(z)
    assert abs(weights[0] - float(s[0] / (s[0] + s[3]))) < 1e-12 and abs(sum(weights) - 1.0) < 1e-12
    assert P.route(torch.zeros(6, dtype=torch.float64), 3, 3, 2)[0] == [0, 1, 2]      # equals: the lower index
    assert P.route(torch.tensor([0.1, 0.3, 0.2], dtype=torch.float64), 2, 3, 2)[0] == [1, 2]    # groups of one
    assert P.is_close_call(z, [3, 4], {"router": {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}}}, 0.0)
    assert not P.is_close_call(z, [0, 3], {"router": {"experts": 6, "top": 2, "groups": {"count": 2, "keep": 1}}}, 0.1)


def test_gelu_and_norm():
    z = torch.tensor([-3.0, -0.5, 0.0, 0.5, 3.0], dtype=torch.float64)
    exact = 0.5 * z * (1 + torch.erf(z / math.sqrt(2)))
    assert torch.allclose(P.gelu_tanh(z), exact, atol=3e-3) and float(P.gelu_tanh(z)[2]) == 0.0
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(P.norm_around_zero(x, torch.zeros(2, dtype=torch.float64), 0.0), x / math.sqrt(12.5))
    assert torch.allclose(P.norm_around_zero(x, torch.tensor([1.0, -1.0], dtype=torch.float64), 0.0),
                          torch.tensor([[2 * 3 / math.sqrt(12.5), 0.0]], dtype=torch.float64))


@pytest.mark.parametrize("kind,mixer,far", [
    ("attention", _windowed(2, 1, 8, 5, 2, 4), 2), ("latent_attention", _latent(2, 4, 2, 6, 5, 5), 0), ("attention_2", _chunked(2, 1, 8, 6, 4), 7)])
def test_a_token_out_of_sight_changes_nothing_and_one_in_sight_does(kind, mixer, far):
    """One layer: the output at position 10 does not change with the input at a position it does not see (for the
    first kind, the first position that is not kept), and does with its neighbour that it sees."""
    cfg = one_layer(kind, mixer, width=16)
    W = _weights(cfg)
    torch.manual_seed(0)
    h = torch.randn(11, 16, dtype=torch.float64)
    base = P.mixer(kind, h, list(range(11)), W, "l0.mix.", mixer, 1e-6)[10]
    for j, seen in ((far, False), (far - 1 if kind == "attention" else 6 if kind == "latent_attention" else 8, True)):
        h2 = h.clone()
        h2[j] += 1.0
        moved = P.mixer(kind, h2, list(range(11)), W, "l0.mix.", mixer, 1e-6)[10]
        assert (not torch.equal(moved, base)) == seen, f"{kind}: position {j}"


def test_values_are_the_keys_before_norm_and_rotation():
    """With one head, a window of the token itself and nothing kept, a token attends to itself only, so the mixer is
    ``W_o (W_k h + b_k)`` whatever norms and rotation do to queries and keys."""
    mixer = _windowed(1, 1, 8, 1, 0, 8)
    cfg = one_layer("attention", mixer, width=16)
    W = _weights(cfg)
    h = torch.randn(5, 16, dtype=torch.float64)
    got = P.mixer_attention(h, list(range(5)), W, "l0.mix.", mixer, 1e-6)
    assert torch.allclose(got, (h @ W["l0.mix.k"].T + W["l0.mix.k.b"]) @ W["l0.mix.o"].T)


def test_shared_expert_has_a_gate_per_token():
    mlp = _moe(2, 2, 8, shared=6)
    cfg = one_layer("attention_2", _chunked(1, 1, 8, 8, 4), mlp, width=16)
    W = _weights(cfg)
    h = torch.randn(3, 16, dtype=torch.float64)
    full = P.ff_experts(h, W, "l0.mlp.", mlp)
    W2 = dict(W)
    W2["l0.mlp.shared.sg"] = W["l0.mlp.shared.sg"] - 100.0 * h[1:2] / (h[1] ** 2).sum()      # closes the gate of token 1 only
    closed = P.ff_experts(h, W2, "l0.mlp.", mlp)
    routed_only = P.ff_experts(h, W, "l0.mlp.", {k: v for k, v in mlp.items() if k != "shared"})
    assert torch.allclose(closed[1], routed_only[1], atol=1e-12) and float((full[1] - routed_only[1]).abs().max()) > 1e-7
