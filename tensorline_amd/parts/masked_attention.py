"""Grouped-query softmax attention over the paged cache whose sight is cut by a mask, with the options that
designs combine around it:

* ``mask``: which earlier keys a token at position p sees besides itself: ``{"kind": "window", "size": w,
  "keep_first": f}``: the ``w - 1`` keys before it, and the first ``f`` keys of the sequence however far the window
  has moved (they keep their own positions); ``{"kind": "chunk", "size": c}``: the keys from the last multiple of
  ``c`` at or below p on, positions counted from the start of the sequence; None: all of them;
* ``values``: "proj" (a value projection ``v`` of ``vdim`` per key head) or "keys": there is no value projection,
  a key head's values are its keys as projected (with bias), before norm and rotation;
* ``qk_norm``: every query and key head is RMS-normed over its ``dim`` values with a weight per dimension that all
  heads share (``q.norm``, ``k.norm`` [dim]), before rotation;
* ``rot`` = {dims, base, scaling or None}: neighbouring pairs (2i, 2i + 1) of a head's first ``dims`` dimensions are
  turned by ``pos * f_i``, ``f_i = base^(-2i / dims)`` (blended YaRN's way with ``scaling``); None: positions do not
  enter the scores;
* ``gate``: "head": head h's output is multiplied by ``sigmoid(W_g h)_h`` (``g`` [heads, width]); "column": every
  output column by its own gate (``g`` [heads * vdim, width]); None.  The gate reads the mixer's input;
* ``bias``: q, k (and v) carry biases (``.b``).

Tensors under the prefix: q, k, (v), (g), o, (q.norm, k.norm).  One fused product gives q | k | (v) | (gate) in
float32; one kernel does everything between it and attention (norms, rotation, the cache writes); attention runs
on the framework's paged kernels, which know the masks; the cache manager is told what may be given back while the
request lives (the pages a window or a chunk has passed, but never those of the kept first keys).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.attention import PagedAttention
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_mixer
from tensorline_amd.parts.rotary import yarn_frequencies
from tensorline_amd.parts.spec import CacheNeed, TensorDecl, keys_and_values

MASK_KINDS = ("window", "chunk")


def read_mask(prefix: str, mask: dict | None) -> tuple[int, int, int]:
    """(window, keep_first, chunk) of a ``mask`` parameter; zeros for what it does not have."""
    if not mask:
        return 0, 0, 0
    kind, size = mask.get("kind", "window"), int(mask.get("size", 0))
    if kind not in MASK_KINDS or size <= 0:
        raise ValueError(f"{prefix}: mask {mask!r} must be of kind {' or '.join(MASK_KINDS)} with a positive size")
    first = int(mask.get("keep_first", 0) or 0)
    if first < 0 or (first and kind != "window"):
        raise ValueError(f"{prefix}: keep_first comes with a window and is not negative")
    return (size, first, 0) if kind == "window" else (0, 0, size)


@register_mixer("masked_attention")
class MaskedAttention(Part):
    def __init__(self, hidden_size, prefix, dtype, device, heads: int, kv_heads: int, dim: int, scale: float,
                 vdim: int | None = None, values: str = "proj", mask: dict | None = None, qk_norm: bool = False,
                 eps: float = 1e-6, rot: dict | None = None, gate: str | None = None, bias: bool = False):
        super().__init__(hidden_size, prefix, dtype, device)
        self.heads, self.kv_heads, self.dim = int(heads), int(kv_heads), int(dim)
        self.vdim = self.dim if vdim is None else int(vdim)
        if values not in ("proj", "keys") or gate not in (None, "head", "column"):
            raise ValueError(f"{prefix}: values {values!r} must be 'proj' or 'keys', gate {gate!r} 'head', 'column' or None")
        self.values_from_keys = values == "keys"
        if min(self.heads, self.kv_heads, self.dim, self.vdim) <= 0 or self.heads % self.kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads of {dim} and {kv_heads} key/value heads of {self.vdim} do not fit")
        if self.values_from_keys and self.vdim != self.dim:
            raise ValueError(f"{prefix}: values that are the keys have the keys' size, not {self.vdim}")
        self.kernel_dim = -(-max(self.dim, self.vdim) // 16) * 16
        if not kernels.attention_takes_head_dim(self.kernel_dim):
            raise ValueError(f"{prefix}: a head size of {max(self.dim, self.vdim)} is not served: the attention kernels "
                             "take up to 256")
        self.scale, self.eps = float(scale), float(eps)
        if self.scale <= 0.0:
            raise ValueError(f"{prefix}: the score scale {scale} must be positive")
        self.window, self.keep_first, self.chunk = read_mask(prefix, mask)
        self.qk_norm, self.gate = bool(qk_norm), gate
        self.freq, self.mag = None, 1.0
        if rot:
            dims = int(rot["dims"])
            if dims <= 0 or dims % 2 or dims > self.dim:
                raise ValueError(f"{prefix}: rot.dims {dims} must be even and within the head size {self.dim}")
            freq, self.mag = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
            self.freq = freq.to(device)
        mk = lambda s, n_in, n_out, b: Linear(prefix + s, n_in, n_out, b, weight_name=prefix + s, bias_name=prefix + s + ".b")
        self._projs = [mk("q", hidden_size, self.heads * self.dim, bias), mk("k", hidden_size, self.kv_heads * self.dim, bias)]
        if not self.values_from_keys:
            self._projs.append(mk("v", hidden_size, self.kv_heads * self.vdim, bias))
        self.gate_cols = 0 if gate is None else self.heads if gate == "head" else self.heads * self.vdim
        self._gate = mk("g", hidden_size, self.gate_cols, False) if gate else None
        self.qkv_cols = sum(p.out_features for p in self._projs)
        self.qkv: Linear | None = None
        self.o_proj = mk("o", self.heads * self.vdim, hidden_size, False)
        self.q_norm = self.k_norm = None

    # ---- weights -----------------------------------------------------------------------
    def tensors(self):
        out = {}
        for p in self._projs + [self.o_proj] + ([self._gate] if self._gate else []):
            out.update(p.tensors())
        if self.qk_norm:
            out[self.prefix + "q.norm"] = TensorDecl((self.dim,), "one_plus_normal", 0.1, "float32")
            out[self.prefix + "k.norm"] = TensorDecl((self.dim,), "one_plus_normal", 0.1, "float32")
        return out

    def load(self, get: TensorGetter) -> None:
        parts = list(self._projs) + ([self._gate] if self._gate else [])
        for p in parts + [self.o_proj]:
            p.load(get)
        D = self.kernel_dim
        if D != self.vdim:
            # attention leaves D columns per head: zero columns of o for the padding, and a column gate's rows likewise
            w = self.o_proj.weight
            wide = w.new_zeros(w.shape[0], self.heads, D)
            wide[:, :, :self.vdim] = w.view(w.shape[0], self.heads, self.vdim)
            self.o_proj.weight, self.o_proj.in_features = wide.view(w.shape[0], self.heads * D), self.heads * D
            if self.gate == "column":
                g = self._gate.weight
                wide = g.new_zeros(self.heads, D, g.shape[1])
                wide[:, :self.vdim] = g.view(self.heads, self.vdim, g.shape[1])
                self._gate.weight, self._gate.out_features = wide.view(self.heads * D, g.shape[1]), self.heads * D
                self.gate_cols = self.heads * D
        self.qkv = fuse_linears(self.prefix + "qkv", parts)
        for p in parts:
            p.weight = p.bias = None
        self.o_proj.prepare()
        if self.qk_norm:
            self.q_norm, self.k_norm = get(self.prefix + "q.norm"), get(self.prefix + "k.norm")

    def weight_tensors(self):
        return self.qkv.tensors_kept() + self.o_proj.tensors_kept() + [t for t in (self.q_norm, self.k_norm, self.freq) if t is not None]

    def library_products(self):
        return [(lin.weight, torch.float32) for lin in (self.qkv, self.o_proj) if lin.weight is not None]

    # ---- what it keeps -------------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        return keys_and_values(self.kv_heads, self.kernel_dim, self.window, self.keep_first, self.chunk)

    def state_need(self):
        return None

    step_vectors = staticmethod(PagedAttention.step_vectors)

    # ---- one step ------------------------------------------------------------------------
    def forward(self, h, ctx, cache):
        keys, values = cache.planes["k"], cache.planes["v"]
        proj = self.qkv(h, out_dtype=torch.float32)
        q = kernels.head_norm_rotate_store(proj, ctx.pos, self.q_norm, self.k_norm, self.eps, self.freq, self.mag, keys, values,
                                           cache.slots, self.heads, self.kv_heads, self.dim, self.vdim, self.values_from_keys,
                                           self.dtype)
        o = kernels.paged_attention(q, keys, values, cache.tables, ctx.seq_of_token, ctx.pos, self.heads, self.kv_heads,
                                    self.kernel_dim, self.scale, window=self.window, keep_first=self.keep_first,
                                    chunk=self.chunk, q_start=ctx.q_start, ctx_start=ctx.ctx_start, plan=ctx.facts,
                                    single_seqs=ctx.extra.get("attention.single_seqs"))
        if self.gate:
            kernels.head_gate(o, proj[:, self.qkv_cols:self.qkv_cols + self.gate_cols], self.gate_cols)
        return self.o_proj(o, out_dtype=torch.float32)
