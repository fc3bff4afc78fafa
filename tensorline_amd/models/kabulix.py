"""``Kabulix``: how its configuration turns into layers.

A pre-norm decoder (``x <- x + mixer(norm1(x))``, ``x <- x + ff(norm2(x))``, float32 stream) whose RMS norms store
their weights around zero (``x / rms(x) * (1 + w)``).  Each layer has one of three mixers:

* ``attention``: grouped heads; q and k with biases; no value projection, a key head's values are its keys as
  projected; q and k normed per head with a weight all heads share; neighbouring pairs of part of a head turned by
  the position; a sliding window beside which the first tokens of the sequence stay in sight;
* ``latent_attention``: one normed latent and one turned key part cached per token, keys and values of all heads
  made from the latent; a sliding window; YaRN's frequencies; a gate on every output column;
* ``attention_2``: grouped heads, no biases, no positions in the scores; a token sees the tokens of its own chunk
  of positions up to itself; a gate per head.

Feed-forwards: ``W_down (gelu_tanh(W_gate h) * W_up h)``, or routed experts ``W_down (silu(W_gate h) * W_up h)``
chosen among the best groups of experts by ``sigmoid(W_router h)`` and weighted by those scores over their sum,
plus a shared expert times ``sigmoid(W_sg h)``; or none.  The head is the embedding table.  Tensor names:
``embed``, ``l<i>.norm1`` / ``.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``, ``final.norm``.
"""
from __future__ import annotations

from tensorline_amd.config.kabulix_config import KabulixConfig
from tensorline_amd.config.registry import Architecture, register_architecture
from tensorline_amd.parts.spec import LayerSpec, ModelSpec, PartSpec


def _mixer(cfg: KabulixConfig, layer: dict) -> PartSpec:
    m, kind = layer["mixer"], layer["type"]
    mask = m.get("mask")
    if kind == "attention":
        return PartSpec("masked_attention", {
            "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "scale": m["scale"], "values": "keys",
            "mask": {"kind": "window", "size": mask["size"], "keep_first": mask.get("keep_first", 0)} if mask else None,
            "qk_norm": True, "eps": cfg.norm_eps, "rot": m.get("rot"), "gate": None, "bias": True}, prefix="mix.")
    if kind == "latent_attention":
        return PartSpec("latent_attention", {
            "heads": m["heads"], "dim": m["dim"], "rot_dim": m["rot_dim"], "vdim": m["vdim"], "kv_rank": m["kv_rank"],
            "scale": m["scale"], "rot": m["rot"], "eps": cfg.norm_eps, "window": mask["size"] if mask else 0,
            "gate": "column", "rot_layout": "pairs"}, prefix="mix.")
    return PartSpec("masked_attention", {
        "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"], "vdim": m["vdim"], "scale": m["scale"],
        "values": "proj", "mask": {"kind": "chunk", "size": mask["size"]} if mask else None, "qk_norm": False,
        "rot": None, "gate": "head", "bias": False}, prefix="mix.")


def _feed_forward(mlp: dict | None) -> PartSpec | None:
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return PartSpec("swiglu", {"intermediate_size": mlp["ff"], "names": ("gate", "up", "down"),
                                   "activation": "gelu_tanh"}, prefix="mlp.")
    router = mlp["router"]
    groups = router.get("groups") or {"count": 1, "keep": 1}
    shared = mlp.get("shared")
    return PartSpec("routed_experts", {
        "experts": router["experts"], "top": router["top"], "ff": mlp["expert"]["ff"], "weighting": "sigmoid_grouped",
        "groups": groups["count"], "keep_groups": groups["keep"], "router_bias": False, "activation": "swiglu",
        "shared": {"ff": shared["ff"], "gate": True} if shared else None}, prefix="mlp.")


def kabulix_spec(cfg: KabulixConfig) -> ModelSpec:
    norm = lambda name: PartSpec("rmsnorm", {"eps": cfg.norm_eps, "name": name, "around_zero": True})
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = _feed_forward(layer.get("mlp"))
        layers.append(LayerSpec(prefix=f"l{i}.", mixer=_mixer(cfg, layer), feed_forward=ffn, mixer_norm=norm("norm1"),
                                feed_forward_norm=norm("norm2") if ffn is not None else None, block="prenorm_token_input"))
    spec = ModelSpec(
        hidden_size=cfg.hidden_size, vocab_size=cfg.vocab_size, embedding=PartSpec("token_embedding", {"name": "embed"}),
        layers=tuple(layers), final_norm=norm("final.norm"), head=PartSpec("lm_head", {"name": "head", "tied": True}),
        max_position=cfg.max_position_embeddings, eos_token_ids=tuple(cfg.eos_token_id))
    spec.validate()
    return spec


KABULIX = register_architecture(Architecture("Kabulix", KabulixConfig, kabulix_spec), replace=True)
