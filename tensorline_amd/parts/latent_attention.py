"""Attention over a compressed latent: what is cached per token is one normed latent vector and
one rotated key part that all heads share, not keys and values per head.

Per token, from the mixer's input h (H heads; per head ``dim`` plain and ``rot_dim`` rotated
query/key dimensions, ``vdim`` value dimensions; latent size ``kv_rank``):

    q_h  = (W_q h)_h = [q_h^plain | q_h^rot]               c = rmsnorm(first kv_rank rows of W_dkv h) * w
    k^rot = last rot_dim rows of W_dkv h                   k_h^plain = (W_uk c)_h,   v_h = (W_uv c)_h
    score_h(i, j) = (q_h^plain(i) . k_h^plain(j) + R(q_h^rot(i)) . R(k^rot(j))) * scale,  j <= i
    out = W_o concat_h( sigmoid((W_g h)_h) * softmax_j(score_h) v_h )

Options: ``window`` (a token sees itself and the ``window - 1`` keys before it), ``gate`` "column" (every output
column has a gate of its own, ``g`` [heads * vdim, width], instead of one per head), ``rot_layout`` "pairs" (the
rotation turns neighbours (2i, 2i + 1) instead of (i, i + rot_dim / 2)).

The expansion of keys and values never happens here.  Because k_h^plain(j) = U_h c(j) with U_h the
head's rows of W_uk, the plain part of a score is (U_h^T q_h^plain(i)) . c(j): the query is taken
into the latent space once per token, the attention kernel then sees H query heads over ONE shared
key/value head whose key is [c | R(k^rot)] and whose value is c, and the head's rows of W_uv are
applied to the weighted sum of latents afterwards.  That is the paged attention the framework
already has, with ``num_kv_heads`` 1 and a head size of kv_rank + rot_dim (rounded up to 32, 64, 128 or 256).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.attention import PagedAttention
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_mixer
from tensorline_amd.parts.rotary import yarn_frequencies
from tensorline_amd.parts.spec import CacheNeed, TensorDecl, keys_and_values


@register_mixer("latent_attention")
class LatentAttention(Part):
    """Parameters: ``heads``, ``dim`` (plain query/key dimensions per head), ``rot_dim`` (rotated
    ones; the rotation turns all of them), ``vdim``, ``kv_rank``, ``scale`` (applied to the score as
    it is), ``rot`` = {base, dims, scaling} with ``scaling`` = {factor, original, fast, slow} or None,
    ``eps`` of the latent's RMS norm, ``window``, ``gate`` ("head" or "column"), ``rot_layout`` ("halves" or
    "pairs").  Tensors under the prefix: q, dkv, dkv.norm, uk, uv, g, o."""

    def __init__(self, hidden_size, prefix, dtype, device, heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int,
                 scale: float, rot: dict, eps: float, window: int = 0, gate: str = "head", rot_layout: str = "halves"):
        super().__init__(hidden_size, prefix, dtype, device)
        if gate not in ("head", "column") or rot_layout not in ("halves", "pairs"):
            raise ValueError(f"{prefix}: gate {gate!r} must be 'head' or 'column', rot_layout {rot_layout!r} 'halves' or 'pairs'")
        self.window, self.gate, self.rot_layout = int(window or 0), gate, rot_layout
        self.heads, self.dim, self.rot_dim, self.vdim, self.rank = int(heads), int(dim), int(rot_dim), int(vdim), int(kv_rank)
        self.scale, self.eps = float(scale), float(eps)
        if int(rot.get("dims", self.rot_dim)) != self.rot_dim or self.rot_dim % 2:
            raise ValueError(f"{prefix}: the rotation turns {rot.get('dims')} dimensions, the rotated part has {self.rot_dim}; "
                             "they must be equal and even")
        # the width of a cached row: latent, rotated key part, zeros up to the next head size that the
        # matrix-core attention kernels take (32, 64, 128, 256)
        need = self.rank + self.rot_dim
        self.cache_dim = next((d for d in kernels.MFMA_HEAD_DIMS if d >= need), 0)
        self.wide = not self.cache_dim
        if self.wide:
            # wider than those kernels take: rows in steps of 16 and the plain wide-row attention (slow;
            # it keeps such a model served)
            self.cache_dim = -(-need // 16) * 16
            if self.cache_dim > kernels.WIDE_ROW_MAX:
                raise ValueError(f"{prefix}: kv_rank + rot_dim = {need} is not served: cached rows of up to {kernels.WIDE_ROW_MAX}")
        freq, self.mag = yarn_frequencies(self.rot_dim, float(rot["base"]), rot.get("scaling"))
        self.freq = freq.to(device)
        H = self.heads
        n = lambda s: prefix + s
        self._q = Linear(n("q"), hidden_size, H * (self.dim + self.rot_dim), False, weight_name=n("q"))
        self._dkv = Linear(n("dkv"), hidden_size, self.rank + self.rot_dim, False, weight_name=n("dkv"))
        self.gate_cols = H if gate == "head" else H * self.vdim
        self._g = Linear(n("g"), hidden_size, self.gate_cols, False, weight_name=n("g"))
        self.proj: Linear | None = None
        self.o_proj = Linear(n("o"), H * self.vdim, hidden_size, False, weight_name=n("o"))
        self.norm_w = self.uk_t = self.uv = None

    def tensors(self):
        out = {}
        for p in (self._q, self._dkv, self._g, self.o_proj):
            out.update(p.tensors())
        out[self.prefix + "dkv.norm"] = TensorDecl((self.rank,), "one_plus_normal", 0.1, "float32")
        out[self.prefix + "uk"] = TensorDecl((self.heads * self.dim, self.rank), "normal", 0.05, "compute")
        out[self.prefix + "uv"] = TensorDecl((self.heads * self.vdim, self.rank), "normal", 0.05, "compute")
        return out

    def load(self, get: TensorGetter) -> None:
        for p in (self._q, self._dkv, self._g, self.o_proj):
            p.load(get)
        if self.rot_layout == "pairs":
            # The kernel turns (i, i + rot_dim / 2).  A score is a sum over the rotated dimensions, so it does not
            # change when queries and keys are reordered alike: the rows that make the rotated dimensions are put
            # in the order evens, then odds, which brings neighbours (2i, 2i + 1) to the places (i, i + rot_dim / 2).
            r, step = self.rot_dim, self.dim + self.rot_dim
            order = torch.cat([torch.arange(0, r, 2), torch.arange(1, r, 2)])
            rows = torch.arange(self.heads * step).view(self.heads, step)
            rows[:, self.dim:] = rows[:, self.dim:][:, order]
            self._q.weight = self._q.weight.index_select(0, rows.reshape(-1).to(self._q.weight.device)).contiguous()
            rows = torch.arange(self.rank + r)
            rows[self.rank:] = rows[self.rank:][order]
            self._dkv.weight = self._dkv.weight.index_select(0, rows.to(self._dkv.weight.device)).contiguous()
        self.proj = fuse_linears(self.prefix + "q_dkv_g", [self._q, self._dkv, self._g])
        for p in (self._q, self._dkv, self._g):
            p.weight = None
        self.o_proj.prepare()
        self.norm_w = get(self.prefix + "dkv.norm")
        H, d, dv, r = self.heads, self.dim, self.vdim, self.rank
        # per head: U_h^T [rank, dim] takes a plain query part into the latent space, V_h [vdim, rank]
        # takes a weighted sum of latents to the head's values
        self.uk_t = get(self.prefix + "uk").view(H, d, r).transpose(1, 2).contiguous()
        self.uv = get(self.prefix + "uv").view(H, dv, r).contiguous()

    def weight_tensors(self):
        return self.proj.tensors_kept() + self.o_proj.tensors_kept() + [self.norm_w, self.uk_t, self.uv]

    def library_products(self):
        return [(self.o_proj.weight, torch.float32)]

    def cache_need(self) -> CacheNeed | None:
        return keys_and_values(1, self.cache_dim, self.window)

    def state_need(self):
        return None

    step_vectors = staticmethod(PagedAttention.step_vectors)

    def forward(self, h, ctx, cache):
        T, H, D = h.shape[0], self.heads, self.cache_dim
        keys, values = cache.planes["k"], cache.planes["v"]
        proj = self.proj(h, out_dtype=torch.float32)
        q_plain, q_lat = kernels.latent_prepare(proj, ctx.pos, self.freq, self.mag, self.norm_w, self.eps, cache.slots,
                                                keys, values, H, self.dim, self.rot_dim, self.rank)
        kernels.batched_linear(q_plain.view(T, H, self.dim), self.uk_t, q_lat.view(T, H, D)[:, :, :self.rank])
        if self.wide:
            o_lat = kernels.wide_row_attention(q_lat, keys, cache.tables, ctx.seq_of_token, ctx.pos, H, self.scale,
                                               window=self.window)
        else:
            o_lat = kernels.paged_attention(q_lat, keys, values, cache.tables, ctx.seq_of_token, ctx.pos, H, 1, D, self.scale,
                                            window=self.window, q_start=ctx.q_start, ctx_start=ctx.ctx_start, plan=ctx.facts,
                                            single_seqs=ctx.extra.get("attention.single_seqs"))
        o = torch.empty(T, H * self.vdim, dtype=o_lat.dtype, device=o_lat.device)
        kernels.batched_linear(o_lat.view(T, H, D)[:, :, :self.rank], self.uv, o.view(T, H, self.vdim))
        gate0 = H * (self.dim + self.rot_dim) + self.rank + self.rot_dim
        kernels.head_gate(o, proj[:, gate0:gate0 + self.gate_cols], self.gate_cols)
        return self.o_proj(o, out_dtype=torch.float32)
