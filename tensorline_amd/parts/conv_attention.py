"""Attention whose queries, keys and values pass a short causal convolution over time right after
their projection, over the framework's paged cache, in two kinds:

* ``conv_attention``: grouped-query softmax attention with an optional rotation of neighbouring pairs
  (YaRN's frequencies) over the first ``rot.dims`` dimensions of a head, an optional window, an optional
  output gate ``sigmoid(W_g h)`` on the concatenated heads, biases on q/k/v (``bias``) and on the output
  projection (``out_bias``);
* ``differential_attention``: every head has two maps (a head's query rows, and a key head's rows, are those of map 1
  followed by those of map 2) over the same values; ``o = a1 - lambda a2`` with ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) +
  diff``, one number per layer, then ``o / rms(o) * (1 - diff)`` per head.  No rotation.

Both: tensors ``q``, ``k``, ``v`` (``.b`` biases, ``.conv`` taps [channels, taps]), ``o``; ``kv_proj`` False
for a layer that reads the keys and values another layer cached (it has queries only); ``window`` is what
a token sees, ``retain`` what the cache keeps (the widest window of the layers that read it).

What a request keeps: the cache pages (keys after convolution and rotation, values after convolution) and,
in its state slot, the last ``taps - 1`` projected rows of q, k and v ahead of the convolution, float32.

The two maps run on the same attention kernels as everything else: as ``2 heads`` query heads over
``2 kv_heads`` key heads, the query heads put in the order (key/value head, map, place in the group) when
the weights are loaded, so that the kernels' grouping finds map m of a group at key head ``2 g + m``; the
values are cached once per map.
"""
from __future__ import annotations

import math

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_mixer
from tensorline_amd.parts.rotary import yarn_frequencies
from tensorline_amd.parts.spec import CacheNeed, StateNeed, TensorDecl, keys_and_values


def _pad_rows(t: torch.Tensor, heads: int, size: int, padded: int) -> torch.Tensor:
    """[heads * size, ...] -> [heads * padded, ...]: every head's rows followed by zero rows."""
    if padded == size:
        return t
    wide = t.new_zeros(heads, padded, *t.shape[1:])
    wide[:, :size] = t.view(heads, size, *t.shape[1:])
    return wide.view(heads * padded, *t.shape[1:])


class _ConvAttention(Part):
    maps = 1          # attention maps per head: queries and keys have ``maps * dim`` rows per head

    def __init__(self, hidden_size, prefix, dtype, device, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                 conv: int, window: int = 0, retain: int | None = None, bias: bool = True, out_bias: bool = False,
                 kv_proj: bool = True, gate: bool = False):
        super().__init__(hidden_size, prefix, dtype, device)
        self.heads, self.kv_heads, self.dim, self.vdim = int(heads), int(kv_heads), int(dim), int(vdim)
        if min(self.heads, self.kv_heads, self.dim, self.vdim) <= 0 or self.heads % self.kv_heads:
            raise ValueError(f"{prefix}: {heads} query heads of {dim} and {kv_heads} key/value heads of {vdim} do not fit")
        self.kernel_dim = -(-max(self.dim, self.vdim) // 16) * 16
        if not kernels.attention_takes_head_dim(self.kernel_dim):
            raise ValueError(f"{prefix}: a head size of {max(self.dim, self.vdim)} is not served: the attention kernels "
                             "take up to 256")
        self.scale, self.taps_n = float(scale), int(conv)
        if not 1 <= self.taps_n <= kernels.CONV_MAX_TAPS:
            raise ValueError(f"{prefix}: a convolution of {conv} taps is not served (1 to {kernels.CONV_MAX_TAPS})")
        self.window = int(window or 0)
        self.retain = self.window if retain is None else int(retain)
        if self.retain and (not self.window or self.window > self.retain):
            raise ValueError(f"{prefix}: a window of {self.window or 'all'} tokens looks further back than the {self.retain} the cache keeps")
        self.kv_proj, self.has_gate = bool(kv_proj), bool(gate)
        self.q_heads, self.k_heads = self.maps * self.heads, self.maps * self.kv_heads      # as the kernels see them
        mk = lambda s, n_in, n_out, b: Linear(prefix + s, n_in, n_out, b, weight_name=prefix + s, bias_name=prefix + s + ".b")
        self._projs = [mk("q", hidden_size, self.q_heads * self.dim, bias)]
        if self.kv_proj:
            self._projs += [mk("k", hidden_size, self.k_heads * self.dim, bias), mk("v", hidden_size, self.kv_heads * self.vdim, bias)]
        self._gate = mk("g", hidden_size, self.heads * self.vdim, False) if self.has_gate else None
        self.channels = sum(p.out_features for p in self._projs)
        self.qkv: Linear | None = None
        self.o_proj = mk("o", self.heads * self.vdim, hidden_size, out_bias)
        self.taps: torch.Tensor | None = None
        self.freq, self.mag = None, 1.0

    # ---- weights -----------------------------------------------------------------------
    def tensors(self):
        out = {}
        for p in self._projs:
            out.update(p.tensors())
            out[p.weight_name + ".conv"] = TensorDecl((p.out_features, self.taps_n), "normal", 0.5, "float32")
        for p in (self._gate, self.o_proj):
            if p is not None:
                out.update(p.tensors())
        return out

    def _query_order(self) -> torch.Tensor | None:
        """Rows of the query projection in the order the kernels want them, or None (as stored)."""
        return None

    def _pads_output(self) -> bool:
        """Whether what reaches the output projection has ``kernel_dim`` columns per head."""
        return True

    def load(self, get: TensorGetter) -> None:
        taps = []
        for p in self._projs:
            p.load(get)
            taps.append(get(p.weight_name + ".conv"))
        order = self._query_order()
        if order is not None:
            q = self._projs[0]
            order = order.to(q.weight.device)
            q.weight = q.weight.index_select(0, order).contiguous()
            if q.bias is not None:
                q.bias = q.bias.index_select(0, order).contiguous()
            taps[0] = taps[0].index_select(0, order)
        self.taps = torch.cat(taps, dim=0).t().contiguous()        # [taps, channels]: a tap's weights in a row
        parts = list(self._projs)
        D = self.kernel_dim
        if self._gate is not None:
            self._gate.load(get)
            self._gate.weight = _pad_rows(self._gate.weight, self.heads, self.vdim, D)    # zero rows gate the padding
            self._gate.out_features = self.heads * D
            parts.append(self._gate)
        self.qkv = fuse_linears(self.prefix + "qkv", parts)
        for p in parts:
            p.weight = p.bias = None
        self.o_proj.load(get)
        if self._pads_output() and D != self.vdim:
            w = self.o_proj.weight
            wide = w.new_zeros(w.shape[0], self.heads, D)
            wide[:, :, :self.vdim] = w.view(w.shape[0], self.heads, self.vdim)
            self.o_proj.weight, self.o_proj.in_features = wide.view(w.shape[0], self.heads * D), self.heads * D
        self.o_proj.prepare()

    def weight_tensors(self):
        return self.qkv.tensors_kept() + self.o_proj.tensors_kept() + [self.taps] + ([self.freq] if self.freq is not None else [])

    def library_products(self):
        return [(lin.weight, torch.float32) for lin in (self.qkv, self.o_proj) if lin is not None and lin.weight is not None]

    # ---- what it keeps -------------------------------------------------------------------
    def cache_need(self) -> CacheNeed:
        return keys_and_values(self.k_heads, self.kernel_dim, self.retain if self.kv_proj else self.window)

    def state_need(self) -> StateNeed:
        return StateNeed((max((self.taps_n - 1) * self.channels, 1),), "float32")

    @staticmethod
    def step_vectors(facts) -> dict:
        singles = kernels.one_token_sequences(facts)
        return {"attention.single_seqs": singles} if singles else {}

    # ---- one step ------------------------------------------------------------------------
    def _attend(self, h, ctx, cache):
        """(projection float32 [T, q | k | v | gate], what attention leaves [T, q_heads * kernel_dim])."""
        keys, values = cache.planes["k"], cache.planes["v"]
        proj = self.qkv(h, out_dtype=torch.float32)
        write = self.kv_proj and cache.write
        if self.kv_proj and not cache.write:
            raise ValueError(f"{self.prefix}: a layer with key and value projections needs a cache of its own")
        q = kernels.conv_rotate_store(proj, self.taps, ctx, cache.state, 0, self.freq, self.mag, keys if write else None,
                                      values if write else None, cache.slots if write else None, self.q_heads,
                                      self.k_heads if write else 0, self.dim, self.kv_heads if write else 0, self.vdim,
                                      self.kernel_dim, self.maps, self.dtype)
        o = kernels.paged_attention(q, keys, values, cache.tables, ctx.seq_of_token, ctx.pos, self.q_heads, self.k_heads,
                                    self.kernel_dim, self.scale, window=self.window, q_start=ctx.q_start,
                                    ctx_start=ctx.ctx_start, plan=ctx.facts,
                                    single_seqs=ctx.extra.get("attention.single_seqs"))
        return proj, o


@register_mixer("conv_attention")
class ConvAttention(_ConvAttention):
    """Parameters: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``conv`` (taps), ``window``, ``retain``,
    ``bias``, ``out_bias``, ``kv_proj``, ``gate``, and ``rot`` = {dims, base, scaling {factor, original, fast, slow}
    or None} or None: neighbours (2i, 2i + 1) of a head's first ``dims`` dimensions are turned by ``pos * f_i``."""

    def __init__(self, hidden_size, prefix, dtype, device, rot: dict | None = None, **kw):
        super().__init__(hidden_size, prefix, dtype, device, **kw)
        if rot:
            dims = int(rot["dims"])
            if dims <= 0 or dims % 2 or dims > self.dim:
                raise ValueError(f"{prefix}: rot.dims {dims} must be even and within the head size {self.dim}")
            freq, self.mag = yarn_frequencies(dims, float(rot["base"]), rot.get("scaling"))
            self.freq = freq.to(device)

    def forward(self, h, ctx, cache):
        proj, o = self._attend(h, ctx, cache)
        if self.has_gate:
            n = self.heads * self.kernel_dim
            kernels.head_gate(o, proj[:, self.channels:self.channels + n], n)       # one gate per column
        return self.o_proj(o, out_dtype=torch.float32)


@register_mixer("differential_attention")
class DifferentialAttention(_ConvAttention):
    """Parameters: ``heads``, ``kv_heads``, ``dim``, ``vdim``, ``scale``, ``conv``, ``window``, ``retain``, ``bias``,
    ``kv_proj``, ``diff`` and ``eps`` (of the norm per head).  Tensors besides the projections: ``lq1``, ``lk1``,
    ``lq2``, ``lk2`` [dim]."""
    maps = 2

    def __init__(self, hidden_size, prefix, dtype, device, diff: float, eps: float, **kw):
        super().__init__(hidden_size, prefix, dtype, device, **kw)
        self.diff, self.eps = float(diff), float(eps)
        self.lam = 0.0

    def tensors(self):
        out = super().tensors()
        for name in ("lq1", "lk1", "lq2", "lk2"):
            out[self.prefix + name] = TensorDecl((self.dim,), "normal", 0.3, "float32")
        return out

    def _query_order(self) -> torch.Tensor:
        H, G, d = self.heads, self.kv_heads, self.dim
        R = H // G
        rows = torch.arange(H * 2 * d).view(G, R, 2, d)         # stored: head g R + r, map m
        return rows.permute(0, 2, 1, 3).reshape(-1)             # wanted: key head 2 g + m, place r

    def _pads_output(self) -> bool:
        return False                                            # the two maps are put together without padding

    def load(self, get: TensorGetter) -> None:
        super().load(get)
        l = {n: get(self.prefix + n).to(torch.float32) for n in ("lq1", "lk1", "lq2", "lk2")}
        # one float32 number per layer, from float32 sums and exponentials
        lam = torch.exp((l["lq1"] * l["lk1"]).sum()) - torch.exp((l["lq2"] * l["lk2"]).sum())
        self.lam = float(lam.item()) + self.diff
        if not math.isfinite(self.lam):
            raise ValueError(f"{self.prefix}: the factor between the two maps is not finite")

    def forward(self, h, ctx, cache):
        _, a = self._attend(h, ctx, cache)
        o = kernels.diff_combine(a, self.heads, self.kv_heads, self.vdim, self.kernel_dim, self.lam, self.eps, 1.0 - self.diff)
        return self.o_proj(o, out_dtype=torch.float32)
