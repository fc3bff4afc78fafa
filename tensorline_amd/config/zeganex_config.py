"""Typed configuration of the Zeganex decoder: attention layers of two kinds with short convolutions,
norms on both sides of every branch, a hashed bigram row added to the token embedding.

``config.json`` gives: ``architecture`` "Zeganex", ``vocab``, ``width``, ``norm.eps``, ``residual_mult`` (the
factor on every normed branch output), ``embedding.bigram`` = {buckets, mul_prev, mul_cur}, and ``layers``,
one entry per layer: ``type`` "attention" (two maps per head, subtracted) or "attention_2" (rotation, output
gate), ``mixer`` = {heads, kv_heads, dim, vdim, scale, conv, mask {size}, and diff | rot {dims, base, scaling},
optionally kv_from: the layer whose cached keys and values this one reads}, ``mlp`` = {kind "dense", ff} or
{kind "moe", router {experts, top}, expert {ff}} or null.
"""
from __future__ import annotations

import copy
import json
import os
from dataclasses import dataclass, field
from typing import Any, Mapping

from tensorline_amd.config.model_config import ConfigError

_MIXER_KEYS = ("heads", "kv_heads", "dim", "vdim", "scale", "conv")
LAYER_TYPES = ("attention", "attention_2")


def _positive_int(where: str, d: Any, key: str) -> int:
    v = d.get(key) if isinstance(d, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


@dataclass(frozen=True)
class ZeganexConfig:
    vocab_size: int
    hidden_size: int
    layers: tuple = ()                      # the entries of config.json's ``layers``, checked
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    bigram: tuple[int, int, int] | None = None      # (buckets, mul_prev, mul_cur)
    eos_token_id: tuple[int, ...] = ()
    max_position_embeddings: int = 1 << 30
    architecture: str = "Zeganex"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, hash=False)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "ZeganexConfig":
        vocab, width = _positive_int("", d, "vocab"), _positive_int("", d, "width")
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("config.json: 'layers' must be a non-empty list")
        norm = d.get("norm") or {}
        if "eps" not in norm:
            raise ConfigError("config.json: norm.eps is missing")
        layers = []
        for i, layer in enumerate(raw_layers):
            where = f"layers[{i}]"
            kind, mixer = layer.get("type"), layer.get("mixer")
            if kind not in LAYER_TYPES:
                raise ConfigError(f"config.json: {where}.type {kind!r} is unknown; known: {', '.join(LAYER_TYPES)}")
            if not isinstance(mixer, Mapping):
                raise ConfigError(f"config.json: {where}.mixer is missing")
            for key in _MIXER_KEYS:
                if key not in mixer:
                    raise ConfigError(f"config.json: {where}.mixer.{key} is missing")
            for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                _positive_int(where + ".mixer", mixer, key)
            if mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"config.json: {where}.mixer: {mixer['heads']} heads are not a multiple of {mixer['kv_heads']} kv_heads")
            mask = mixer.get("mask")
            if mask is not None:
                _positive_int(where + ".mixer.mask", mask, "size")
            if kind == "attention" and "diff" not in mixer:
                raise ConfigError(f"config.json: {where}.mixer.diff is missing")
            rot = mixer.get("rot")
            if rot is not None:
                if kind == "attention":
                    raise ConfigError(f"config.json: {where}: a layer of type 'attention' has no rotation")
                _positive_int(where + ".mixer.rot", rot, "dims")
                if "base" not in rot:
                    raise ConfigError(f"config.json: {where}.mixer.rot.base is missing")
                sc = rot.get("scaling")
                if sc is not None:
                    for key in ("factor", "original", "fast", "slow"):
                        if key not in sc:
                            raise ConfigError(f"config.json: {where}.mixer.rot.scaling.{key} is missing")
            src = mixer.get("kv_from")
            if src is not None:
                if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < i:
                    raise ConfigError(f"config.json: {where}.mixer.kv_from {src!r} must name an earlier layer")
                other = raw_layers[src]
                if other.get("type") != kind or other["mixer"].get("kv_from") is not None:
                    raise ConfigError(f"config.json: {where}.mixer.kv_from: layer {src} must be of the same type and cache its own keys")
                for key in ("kv_heads", "dim", "vdim"):
                    if other["mixer"].get(key) != mixer[key]:
                        raise ConfigError(f"config.json: {where}.mixer.kv_from: layer {src} has another {key}")
            mlp = layer.get("mlp")
            if mlp is not None:
                mk = mlp.get("kind")
                if mk == "dense":
                    _positive_int(where + ".mlp", mlp, "ff")
                elif mk == "moe":
                    _positive_int(where + ".mlp.router", mlp.get("router"), "experts")
                    _positive_int(where + ".mlp.router", mlp.get("router"), "top")
                    _positive_int(where + ".mlp.expert", mlp.get("expert"), "ff")
                    if mlp["router"]["top"] > mlp["router"]["experts"]:
                        raise ConfigError(f"config.json: {where}.mlp.router.top exceeds the number of experts")
                else:
                    raise ConfigError(f"config.json: {where}.mlp.kind {mk!r} is unknown; known: dense, moe")
            layers.append(copy.deepcopy(dict(layer)))
        big = (d.get("embedding") or {}).get("bigram")
        bigram = None
        if big is not None:
            _positive_int("embedding.bigram", big, "buckets")
            for key in ("mul_prev", "mul_cur"):
                if isinstance(big.get(key), bool) or not isinstance(big.get(key), int):
                    raise ConfigError(f"config.json: embedding.bigram.{key} must be an integer")
            bigram = (int(big["buckets"]), int(big["mul_prev"]), int(big["mul_cur"]))
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "embedding", "residual_mult", "eos_token_id",
                 "max_position_embeddings"}
        return cls(vocab_size=vocab, hidden_size=width, layers=tuple(layers), norm_eps=float(norm["eps"]),
                   residual_mult=float(d.get("residual_mult", 1.0)), bigram=bigram, eos_token_id=eos_ids,
                   max_position_embeddings=int(d.get("max_position_embeddings", 1 << 30)),
                   extra={k: v for k, v in d.items() if k not in known})

    @classmethod
    def from_json(cls, path: str | os.PathLike) -> "ZeganexConfig":
        p = os.fspath(path)
        if os.path.isdir(p):
            p = os.path.join(p, "config.json")
        with open(p, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps}, "residual_mult": self.residual_mult,
                               "layers": copy.deepcopy(list(self.layers))}
        if self.bigram is not None:
            out["embedding"] = {"bigram": {"buckets": self.bigram[0], "mul_prev": self.bigram[1], "mul_cur": self.bigram[2]}}
        if self.eos_token_id:
            out["eos_token_id"] = list(self.eos_token_id)
        return out
