"""Shared by the Zeganex tests: small configurations (none of them a real model's sizes) and random
weights for the framework and for the plain implementation alike."""
from __future__ import annotations

import copy

import torch

from tensorline_amd.config.zeganex_config import ZeganexConfig

YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}


def _rotary(heads, kv_heads, dim, vdim, conv, window, dims, base=500.0, scaling=None, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv,
         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if dims:
        m["rot"] = {"dims": dims, "base": base, "scaling": scaling}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _two_maps(heads, kv_heads, dim, vdim, conv, window, diff=0.55, scale=None, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "diff": diff,
         "scale": scale if scale is not None else dim ** -0.5}
    if window:
        m["mask"] = {"size": window}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def _moe(experts, top, ff):
    return {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _model(vocab, width, layers, eps=1e-5, mult=0.75, bigram=(251, 31, 7)):
    cfg = {"architecture": "Zeganex", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult, "layers": layers}
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0], "mul_prev": bigram[1], "mul_cur": bigram[2]}}
    return cfg


# both mixers, both feed-forwards and a layer without one, a layer of each kind that reads another's cache (one with
# a narrower window than the layer that writes it, one with a wider), windows on both sides of a page of 16
CFG_A = _model(320, 96, [
    {"type": "attention_2", "mixer": _rotary(4, 2, 24, 40, 3, 21, 8, scaling=YARN), "mlp": _dense(136)},
    {"type": "attention", "mixer": _two_maps(4, 2, 16, 24, 4, 33), "mlp": _moe(6, 2, 40)},
    {"type": "attention_2", "mixer": _rotary(4, 2, 24, 40, 2, 13, 8, scaling=YARN, kv_from=0), "mlp": None},
    {"type": "attention", "mixer": _two_maps(2, 2, 16, 24, 3, 47, diff=0.3, kv_from=1), "mlp": _moe(6, 2, 40)},
])
# sizes that are no multiple of 8, one head, one tap, as many choices as experts, full rotation without scaling, no
# bigram table, the two-map layer first, a window of one page and a window wider than any prompt
CFG_B = _model(131, 72, [
    {"type": "attention", "mixer": _two_maps(3, 1, 10, 7, 1, 8, diff=0.8, scale=0.4), "mlp": _moe(3, 3, 20)},
    {"type": "attention_2", "mixer": _rotary(1, 1, 20, 12, 5, 500, 20, base=50.0), "mlp": _dense(50)},
    {"type": "attention_2", "mixer": _rotary(3, 3, 6, 9, 2, 3, 2, scaling={"factor": 1.5, "original": 16, "fast": 4.0, "slow": 1.0}),
     "mlp": _moe(1, 1, 16)},
], eps=1e-6, mult=1.3, bigram=None)
# head sizes the bfloat16 matrix-core attention takes (32, 64 and 128), no window on one layer, one choice of five
CFG_C = _model(200, 128, [
    {"type": "attention_2", "mixer": _rotary(6, 1, 64, 64, 4, 40, 32, scaling=YARN), "mlp": _moe(8, 2, 16)},
    {"type": "attention", "mixer": _two_maps(4, 2, 32, 64, 3, 17, diff=0.5), "mlp": _moe(5, 1, 48)},
    {"type": "attention_2", "mixer": _rotary(2, 2, 128, 96, 2, 0, 16, base=10000.0, scale=0.05), "mlp": _dense(64)},
    {"type": "attention", "mixer": _two_maps(2, 1, 128, 128, 2, 64, diff=0.1, scale=0.05), "mlp": None},
], mult=0.5, bigram=(1019, 113, 19))
CONFIGS = {"A": CFG_A, "B": CFG_B, "C": CFG_C}


def one_layer(kind: str, mixer: dict, mlp=None, width: int = 64, vocab: int = 50, bigram=None) -> dict:
    return _model(vocab, width, [{"type": kind, "mixer": mixer, "mlp": mlp}], eps=1e-6, mult=1.0, bigram=bigram)


def typed(cfg: dict) -> ZeganexConfig:
    return ZeganexConfig.from_dict(copy.deepcopy(cfg))


def build(cfg: dict, dtype: str, seed: int = 0, device="cuda:0", edit=None):
    """(framework model, plain weights by name in float32).  Both hold the same bfloat16-rounded
    values; ``edit(weights)`` may change them first (the model is then loaded from the edited ones)."""
    from tensorline_amd.config.registry import get_architecture
    from tensorline_amd.engine.loading import TORCH_DTYPE
    from tensorline_amd.models.decoder import DecoderModel
    from tensorline_amd.weights.loader import load_from_getter
    from tensorline_amd.weights.random_init import random_tensor
    config = typed(cfg)
    model = DecoderModel(get_architecture("Zeganex").build_spec(config), TORCH_DTYPE[dtype], device)
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
    """A configuration drawn from ``rng`` (a ``random.Random``): one to five layers of either kind in any order,
    sizes that are and are not multiples of 8 or 16, every head grouping, one to five taps, windows from two
    tokens to none, layers that read an earlier layer's cache, every kind of feed-forward."""
    def divisor(n):
        return rng.choice([d for d in range(1, n + 1) if n % d == 0])

    def mlp():
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            return None
        if kind == "dense":
            return _dense(rng.choice([7, 24, 50, 136]))
        experts = rng.randint(1, 9)
        return _moe(experts, rng.randint(1, experts), rng.choice([8, 20, 36, 64]))

    layers = []
    for i in range(rng.randint(1, 5)):
        kind = rng.choice(["attention", "attention_2"])
        window = rng.choice([0, 2, 5, 16, 17, 31, 48, 70])
        earlier = [j for j, l in enumerate(layers) if l["type"] == kind and "kv_from" not in l["mixer"]]
        if earlier and rng.random() < 0.4:
            src = layers[rng.choice(earlier)]["mixer"]
            heads = src["kv_heads"] * rng.choice([1, 2, 3])
            if kind == "attention":
                m = _two_maps(heads, src["kv_heads"], src["dim"], src["vdim"], rng.randint(1, 5), window, diff=rng.choice([0.2, 0.55, 0.9]),
                              scale=src["scale"], kv_from=layers.index(next(l for l in layers if l["mixer"] is src)))
            else:
                m = copy.deepcopy(src)
                m.update(heads=heads, conv=rng.randint(1, 5), kv_from=layers.index(next(l for l in layers if l["mixer"] is src)))
                m.pop("mask", None)
                if window:
                    m["mask"] = {"size": window}
        else:
            heads = rng.choice([1, 2, 3, 4, 6, 8])
            dim = rng.choice([4, 8, 16, 20, 24, 32, 40, 64, 128])
            vdim = rng.choice([4, 8, 12, 16, 32, 48, 64, 128])
            if kind == "attention":
                m = _two_maps(heads, divisor(heads), dim, vdim, rng.randint(1, 5), window, diff=rng.choice([0.2, 0.55, 0.9]),
                              scale=rng.choice([0.05, 0.125, 0.3]))
            else:
                dims = rng.choice([0] + [d for d in (2, 4, 8, 16, 32, 64, 128) if d <= dim])
                m = _rotary(heads, divisor(heads), dim, vdim, rng.randint(1, 5), window, dims, base=rng.choice([50.0, 10000.0]),
                            scaling=rng.choice([None, YARN, {"factor": 3.0, "original": 512, "fast": 24.0, "slow": 1.5}]),
                            scale=rng.choice([0.05, 0.125, 0.3]))
        layers.append({"type": kind, "mixer": m, "mlp": mlp()})
    return _model(rng.randint(50, 400), rng.choice([24, 36, 50, 64, 72, 100, 128, 200]), layers, eps=rng.choice([1e-5, 1e-6]),
                  mult=rng.choice([0.5, 0.75, 1.0, 1.4]),
                  bigram=rng.choice([None, (rng.choice([13, 251, 1019, 100003]), rng.choice([1, 31, 113, 1000003]), rng.choice([1, 7, 19]))]))
