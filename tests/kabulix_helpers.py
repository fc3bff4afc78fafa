"""Shared by the Kabulix tests: small configurations (none of them a real model's sizes) and random weights for the
framework and for the plain implementation alike."""
from __future__ import annotations

import copy

import torch

from tensorline_amd.config.kabulix_config import KabulixConfig

YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}


def _windowed(heads, kv_heads, dim, window, keep_first, dims, base=500.0, scaling=None, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale if scale is not None else dim ** -0.5,
         "mask": {"size": window, "keep_first": keep_first}}
    if dims:
        m["rot"] = {"dims": dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    return m


def _latent(heads, dim, rot_dim, vdim, rank, window, base=3000.0, scaling=YARN, scale=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": rank,
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": base}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window:
        m["mask"] = {"size": window}
    return m


def _chunked(heads, kv_heads, dim, vdim, chunk, scale=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else dim ** -0.5}
    if chunk:
        m["mask"] = {"size": chunk}
    return m


def _moe(experts, top, ff, groups=None, keep=None, shared=None):
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups, "keep": keep}
    out = {"kind": "moe", "router": router, "expert": {"ff": ff}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _model(vocab, width, layers, eps=1e-5):
    return {"architecture": "Kabulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}


# all three mixers, both feed-forwards and a layer without one; windows and a chunk on both sides of a page of 16
CFG_A = _model(320, 96, [
    {"type": "attention", "mixer": _windowed(4, 2, 24, 21, 3, 8), "mlp": _dense(136)},
    {"type": "latent_attention", "mixer": _latent(3, 16, 8, 24, 40, 13), "mlp": _moe(6, 2, 40, groups=3, keep=2, shared=24)},
    {"type": "attention_2", "mixer": _chunked(4, 2, 24, 40, 19), "mlp": None},
    {"type": "attention", "mixer": _windowed(2, 2, 16, 33, 17, 16, scaling=YARN), "mlp": _moe(8, 3, 40, groups=4, keep=2)},
])
# sizes that are no multiple of 8, one head, as many choices as the kept groups hold, groups of one, every group kept,
# full rotation, a chunk of one page, a window wider than any prompt, no kept first tokens, the chunked layer first
CFG_B = _model(131, 72, [
    {"type": "attention_2", "mixer": _chunked(3, 1, 10, 7, 16, scale=0.4), "mlp": _moe(3, 2, 20, groups=3, keep=2, shared=9)},
    {"type": "attention", "mixer": _windowed(1, 1, 20, 500, 0, 20, base=50.0), "mlp": _dense(50)},
    {"type": "latent_attention", "mixer": _latent(1, 6, 2, 9, 11, 3, scaling={"factor": 1.5, "original": 16, "fast": 4.0, "slow": 1.0}),
     "mlp": _moe(4, 4, 16, groups=2, keep=2)},
    {"type": "attention_2", "mixer": _chunked(3, 3, 6, 9, 2), "mlp": _moe(1, 1, 16)},
], eps=1e-6)
# head sizes the bfloat16 matrix-core attention takes (32, 64 and 128), more kept first tokens than a page holds,
# a latent without scaling and without window, a chunked layer without chunk
CFG_C = _model(200, 128, [
    {"type": "attention", "mixer": _windowed(6, 1, 64, 40, 20, 32, scaling=YARN), "mlp": _moe(8, 2, 16, groups=2, keep=1, shared=32)},
    {"type": "latent_attention", "mixer": _latent(4, 32, 16, 32, 48, 0, scaling=None), "mlp": _moe(5, 1, 48)},
    {"type": "attention_2", "mixer": _chunked(2, 2, 128, 96, 0, scale=0.05), "mlp": _dense(64)},
    {"type": "attention_2", "mixer": _chunked(4, 1, 32, 32, 48), "mlp": None},
    {"type": "attention", "mixer": _windowed(2, 1, 128, 64, 2, 16, base=10000.0, scale=0.05), "mlp": None},
])
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def one_layer(kind: str, mixer: dict, mlp=None, width: int = 64, vocab: int = 50) -> dict:
    return _model(vocab, width, [{"type": kind, "mixer": mixer, "mlp": mlp}], eps=1e-6)


def typed(cfg: dict) -> KabulixConfig:
    return KabulixConfig.from_dict(copy.deepcopy(cfg))


def build(cfg: dict, dtype: str, seed: int = 0, device="cuda:0", edit=None):
    """(framework model, plain weights by name in float32).  Both hold the same bfloat16-rounded
    values; ``edit(weights)`` may change them first (the model is then loaded from the edited ones)."""
    from tensorline_amd.config.registry import get_architecture
    from tensorline_amd.engine.loading import TORCH_DTYPE
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    config = typed(cfg)
    model = DecoderModel(get_architecture("Kabulix").build_spec(config), TORCH_DTYPE[dtype], device)
    w = {name: random_tensor(name, decl, seed, "cpu") for name, decl in model.tensor_decls().items()}
    if edit is not None:
        edit(w)
        for name in w:
            w[name] = w[name].to(torch.bfloat16).to(torch.float32)
    load_from_getter(model, lambda name, decl: w[name], device)
    return model, w


def routed_layers(cfg: dict) -> list[int]:
    return [i for i, layer in enumerate(cfg["layers"]) if (layer.get("mlp") or {}).get("kind") == "moe"]


def random_config(rng) -> dict:
    """A configuration drawn from ``rng`` (a ``random.Random``): one to five layers of the three kinds in any order,
    sizes that are and are not multiples of 8 or 16, every head grouping, windows, kept first tokens and chunks
    from one token to more than a prompt, every kind of feed-forward."""
    def divisor(n):
        return rng.choice([d for d in range(1, n + 1) if n % d == 0])

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return _dense(rng.choice([7, 24, 50, 136]))
        groups = rng.choice([1, 1, 2, 3, 4])
        per = rng.randint(1, 4)
        keep = rng.randint(1, groups)
        return _moe(groups * per, rng.randint(1, keep * per), rng.choice([8, 20, 36, 64]), groups=groups if groups > 1 or rng.random() < 0.5 else None,
                    keep=keep, shared=rng.choice([None, 8, 28]))

    layers = []
    for _ in range(rng.randint(1, 5)):
        kind = rng.choice(["attention", "latent_attention", "attention_2"])
        heads = rng.choice([1, 2, 3, 4, 6, 8])
        scale = rng.choice([0.05, 0.125, 0.3])
        if kind == "attention":
            dim = rng.choice([4, 8, 16, 20, 24, 32, 40, 64, 128])
            dims = rng.choice([0] + [d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim])
            m = _windowed(heads, divisor(heads), dim, rng.choice([1, 2, 5, 16, 17, 31, 48, 70, 400]), rng.choice([0, 0, 1, 3, 16, 21]), dims,
                          base=rng.choice([50.0, 10000.0]), scaling=rng.choice([None, YARN]), scale=scale)
        elif kind == "latent_attention":
            m = _latent(heads, rng.choice([4, 8, 16, 24, 32]), rng.choice([2, 4, 8, 16]), rng.choice([4, 8, 12, 32]), rng.choice([5, 16, 40, 100]),
                        rng.choice([0, 1, 2, 5, 16, 17, 31, 48, 70]), base=rng.choice([50.0, 10000.0]),
                        scaling=rng.choice([None, YARN, {"factor": 3.0, "original": 512, "fast": 24.0, "slow": 1.5}]), scale=scale)
        else:
            m = _chunked(heads, divisor(heads), rng.choice([4, 8, 16, 20, 32, 64, 128]), rng.choice([4, 8, 12, 16, 32, 48, 64, 128]),
                         rng.choice([0, 1, 2, 5, 16, 17, 31, 48, 70]), scale=scale)
        layers.append({"type": kind, "mixer": m, "mlp": mlp()})
    return _model(rng.randint(50, 400), rng.choice([24, 36, 50, 64, 72, 100, 128, 200]), layers, eps=rng.choice([1e-5, 1e-6]))
