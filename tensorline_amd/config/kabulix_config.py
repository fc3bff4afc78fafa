"""Typed configuration of the Kabulix decoder: pre-norm layers whose mixer is one of three kinds of masked
attention, with dense or routed feed-forwards.

``config.json`` gives: ``architecture`` "Kabulix", ``vocab``, ``width``, ``norm.eps`` and ``layers``, one entry per
layer: ``type`` and ``mixer``,

* "attention": {heads, kv_heads, dim, vdim, scale, rot {dims, base, scaling?}, mask {size, keep_first?}};
* "latent_attention": {heads, dim, rot_dim, vdim, kv_rank, scale, rot {dims, base, scaling {factor, original, fast,
  slow}?}, mask {size}?};
* "attention_2": {heads, kv_heads, dim, vdim, scale, mask {size}?};

and ``mlp`` = {kind "dense", ff}, {kind "moe", router {experts, top, groups {count, keep}?}, expert {ff}, shared
{ff}?} or null.
"""
from __future__ import annotations

import copy
import json
import os
from dataclasses import dataclass, field
from typing import Any, Mapping

from tensorline_amd.config.model_config import ConfigError

LAYER_TYPES = ("attention", "latent_attention", "attention_2")
_MIXER_KEYS = {"attention": ("heads", "kv_heads", "dim", "scale"),
               "latent_attention": ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"),
               "attention_2": ("heads", "kv_heads", "dim", "vdim", "scale")}
_INT_KEYS = ("heads", "kv_heads", "dim", "vdim", "rot_dim", "kv_rank")


def _positive_int(where: str, d: Any, key: str) -> int:
    v = d.get(key) if isinstance(d, Mapping) else None
    if isinstance(v, bool) or not isinstance(v, int) or v <= 0:
        raise ConfigError(f"config.json: {where}.{key} must be a positive integer, got {v!r}")
    return v


def _check_rot(where: str, rot: Any, dim: int) -> None:
    if not isinstance(rot, Mapping):
        raise ConfigError(f"config.json: {where}.rot must be an object")
    dims = _positive_int(where + ".rot", rot, "dims")
    if dims % 2 or dims > dim:
        raise ConfigError(f"config.json: {where}.rot.dims {dims} must be even and at most {dim}")
    if "base" not in rot:
        raise ConfigError(f"config.json: {where}.rot.base is missing")
    sc = rot.get("scaling")
    if sc is not None:
        for key in ("factor", "original", "fast", "slow"):
            if key not in sc:
                raise ConfigError(f"config.json: {where}.rot.scaling.{key} is missing")


def _check_mlp(where: str, mlp: Any) -> None:
    mk = mlp.get("kind") if isinstance(mlp, Mapping) else None
    if mk == "dense":
        _positive_int(where, mlp, "ff")
    elif mk == "moe":
        router = mlp.get("router")
        experts, top = _positive_int(where + ".router", router, "experts"), _positive_int(where + ".router", router, "top")
        _positive_int(where + ".expert", mlp.get("expert"), "ff")
        groups = router.get("groups")
        count = keep = 1
        if groups is not None:
            count, keep = _positive_int(where + ".router.groups", groups, "count"), _positive_int(where + ".router.groups", groups, "keep")
            if experts % count or keep > count:
                raise ConfigError(f"config.json: {where}.router: {experts} experts do not form {count} equal groups of which {keep} are kept")
        if top > keep * (experts // count):
            raise ConfigError(f"config.json: {where}.router.top exceeds the experts of the kept groups")
        if mlp.get("shared") is not None:
            _positive_int(where + ".shared", mlp["shared"], "ff")
    else:
        raise ConfigError(f"config.json: {where}.kind {mk!r} is unknown; known: dense, moe")


@dataclass(frozen=True)
class KabulixConfig:
    vocab_size: int
    hidden_size: int
    layers: tuple = ()                      # the entries of config.json's ``layers``, checked
    norm_eps: float = 1e-6
    eos_token_id: tuple[int, ...] = ()
    max_position_embeddings: int = 1 << 30
    architecture: str = "Kabulix"
    extra: Mapping[str, Any] = field(default_factory=dict, compare=False, hash=False)

    @property
    def num_hidden_layers(self) -> int:
        return len(self.layers)

    @classmethod
    def from_dict(cls, d: Mapping[str, Any]) -> "KabulixConfig":
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
            where_m = where + ".mixer"
            for key in _MIXER_KEYS[kind]:
                if key not in mixer:
                    raise ConfigError(f"config.json: {where_m}.{key} is missing")
            for key in _INT_KEYS:
                if key in mixer:
                    _positive_int(where_m, mixer, key)
            if "kv_heads" in mixer and mixer["heads"] % mixer["kv_heads"]:
                raise ConfigError(f"config.json: {where_m}: {mixer['heads']} heads are not a multiple of {mixer['kv_heads']} kv_heads")
            if not float(mixer["scale"]) > 0.0:
                raise ConfigError(f"config.json: {where_m}.scale must be positive")
            mask = mixer.get("mask")
            if mask is not None:
                _positive_int(where_m + ".mask", mask, "size")
                first = mask.get("keep_first", 0)
                if isinstance(first, bool) or not isinstance(first, int) or first < 0 or (first and kind != "attention"):
                    raise ConfigError(f"config.json: {where_m}.mask.keep_first {first!r} must be a non-negative integer, on a layer of type 'attention'")
            if kind == "attention":
                if mixer.get("vdim", mixer["dim"]) != mixer["dim"]:
                    raise ConfigError(f"config.json: {where_m}: the values are the keys, so vdim equals dim")
                if mixer.get("rot") is not None:
                    _check_rot(where_m, mixer["rot"], mixer["dim"])
            elif kind == "latent_attention":
                _check_rot(where_m, mixer["rot"], mixer["rot_dim"])
                if mixer["rot"]["dims"] != mixer["rot_dim"]:
                    raise ConfigError(f"config.json: {where_m}: rot.dims must equal rot_dim")
            elif mixer.get("rot") is not None:
                raise ConfigError(f"config.json: {where}: a layer of type 'attention_2' has no rotation")
            if layer.get("mlp") is not None:
                _check_mlp(where + ".mlp", layer["mlp"])
            layers.append(copy.deepcopy(dict(layer)))
        eos = d.get("eos_token_id")
        eos_ids = () if eos is None else tuple(int(e) for e in eos) if isinstance(eos, (list, tuple)) else (int(eos),)
        known = {"architecture", "architectures", "vocab", "width", "layers", "norm", "eos_token_id", "max_position_embeddings"}
        return cls(vocab_size=vocab, hidden_size=width, layers=tuple(layers), norm_eps=float(norm["eps"]), eos_token_id=eos_ids,
                   max_position_embeddings=int(d.get("max_position_embeddings", 1 << 30)),
                   extra={k: v for k, v in d.items() if k not in known})

    @classmethod
    def from_json(cls, path: str | os.PathLike) -> "KabulixConfig":
        p = os.fspath(path)
        if os.path.isdir(p):
            p = os.path.join(p, "config.json")
        with open(p, "r", encoding="utf-8") as f:
            return cls.from_dict(json.load(f))

    def to_dict(self) -> dict[str, Any]:
        out: dict[str, Any] = {"architecture": self.architecture, "vocab": self.vocab_size, "width": self.hidden_size,
                               "norm": {"eps": self.norm_eps}, "layers": copy.deepcopy(list(self.layers))}
        if self.eos_token_id:
            out["eos_token_id"] = list(self.eos_token_id)
        return out
