"""The plain implementation of the Zeganex decoder: slow, whole-sequence, one function per mechanism.

No cache, no batching, no kernels, no code shared with ``tensorline_amd``.  ``w`` is a dict of
tensors by checkpoint name, ``cfg`` the raw dictionary of config.json.  Everything runs in the dtype
of the tensors given (float32, or float64 for error budgets).  The mixers take the positions of their
rows and what an earlier call left (the convolutions' last inputs, the keys and values seen so far),
so a test can also drive them in portions or one token at a time.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F


# ---- small pieces ------------------------------------------------------------------------------
def rms_divide(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return rms_divide(x, eps) * weight


def short_conv(u, taps, before=None):
    """u [T, C]; taps [C, K], the last column is the current token's; ``before`` [K - 1, C] are the
    inputs ahead of u (zeros at a sequence's start).  Returns (out [T, C], the last K - 1 inputs)."""
    T, C = u.shape
    K = taps.shape[1]
    if before is None:
        before = u.new_zeros(K - 1, C)
    full = torch.cat((before, u), dim=0)                      # row t + K - 1 is u[t]
    out = u.new_zeros(T, C)
    for j in range(K):
        out = out + full[j:j + T] * taps[:, j]
    return out, full[full.shape[0] - (K - 1):]


def bigram_rows(tokens, previous, buckets: int, mul_prev: int, mul_cur: int):
    """Row of the bigram table for every token: a hash of (token before, token); ``previous`` is the
    token ahead of ``tokens[0]`` or None at a sequence's start, which reads the table's last row."""
    rows = []
    for t in tokens:
        rows.append(buckets if previous is None else (previous * mul_prev + t * mul_cur) % buckets)
        previous = t
    return rows


def embed(w, cfg, tokens, previous=None):
    x = w["embed"][torch.tensor(tokens)]
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        rows = bigram_rows(tokens, previous, int(big["buckets"]), int(big["mul_prev"]), int(big["mul_cur"]))
        x = x + w["bigram"][torch.tensor(rows)]
    return x


def yarn_table(dims: int, base: float, scaling: dict | None, dtype=torch.float64):
    """(frequency of each of the dims / 2 pairs, factor on cosine and sine)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return torch.tensor(f, dtype=dtype), 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])
    where = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(where(float(scaling["fast"]))), 0)
    hi = min(math.ceil(where(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return torch.tensor(out, dtype=dtype), 0.1 * math.log(factor) + 1.0


def rotate_pairs(x, positions, rot: dict | None):
    """x [T, heads, d]: neighbours (2i, 2i + 1) of the first rot.dims dimensions turned by the angle
    position * frequency_i; the rest passes."""
    if not rot:
        return x
    dims = int(rot["dims"])
    freq, mag = yarn_table(dims, float(rot["base"]), rot.get("scaling"))
    ang = positions.to(torch.float64)[:, None] * freq[None, :]
    cos, sin = (torch.cos(ang) * mag).to(x.dtype)[:, None, :], (torch.sin(ang) * mag).to(x.dtype)[:, None, :]
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = a * cos - b * sin
    out[..., 1:dims:2] = b * cos + a * sin
    return out


def windowed_softmax_attention(q, k, v, scale, q_pos, k_pos, window):
    """q [Tq, d], k [Tk, d], v [Tk, dv]: position i sees j with 0 <= i - j < window (window 0: all j <= i)."""
    s = (q @ k.T) * scale
    gap = q_pos[:, None] - k_pos[None, :]
    hidden = gap < 0
    if window:
        hidden = hidden | (gap >= window)
    s = s.masked_fill(hidden, float("-inf"))
    return torch.softmax(s, dim=-1) @ v


def _project(h, w, name):
    y = h @ w[name].T
    return y + w[name + ".b"] if name + ".b" in w else y


class MixerMemory:
    """What a mixer of one sequence keeps between calls."""

    def __init__(self):
        self.conv = {}          # name -> last inputs of that convolution
        self.k = self.v = self.pos = None


def _conv_of(name, u, w, mem):
    out, mem.conv[name] = short_conv(u, w[name + ".conv"], mem.conv.get(name))
    return out


def _remember(mem, k, v, pos):
    if mem.k is None:
        mem.k, mem.v, mem.pos = k, v, pos
    else:
        mem.k, mem.v, mem.pos = torch.cat((mem.k, k)), torch.cat((mem.v, v)), torch.cat((mem.pos, pos))


# ---- mixers --------------------------------------------------------------------------------------
def gated_rotary_attention(h, w, p, m, positions, mem: MixerMemory, shared: MixerMemory | None = None):
    """Mixer 'attention_2': projections with biases, short convolutions, rotation of neighbours with
    YaRN's frequencies, a window, softmax, and sigmoid(W_g h) on the heads' outputs before W_o."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = _conv_of(p + "q", _project(h, w, p + "q"), w, mem).view(T, H, d)
    q = rotate_pairs(q, positions, m.get("rot"))
    if shared is None:
        k = _conv_of(p + "k", _project(h, w, p + "k"), w, mem).view(T, G, d)
        v = _conv_of(p + "v", _project(h, w, p + "v"), w, mem).view(T, G, dv)
        _remember(mem, rotate_pairs(k, positions, m.get("rot")), v, positions)
        shared = mem
    window = int((m.get("mask") or {}).get("size", 0))
    out = h.new_zeros(T, H, dv)
    for head in range(H):
        g = head // (H // G)
        out[:, head] = windowed_softmax_attention(q[:, head], shared.k[:, g], shared.v[:, g], float(m["scale"]),
                                                  positions, shared.pos, window)
    out = out.reshape(T, H * dv) * torch.sigmoid(h @ w[p + "g"].T)
    return _project(out, w, p + "o")


def differential_lambda(w, p, diff):
    return (torch.exp((w[p + "lq1"] * w[p + "lk1"]).sum()) - torch.exp((w[p + "lq2"] * w[p + "lk2"]).sum()) + diff).item()


def differential_attention(h, w, p, m, positions, eps, mem: MixerMemory, shared: MixerMemory | None = None):
    """Mixer 'attention': two softmax maps per head over the same values, subtracted with one factor per
    layer, the difference divided by its root mean square and scaled; no rotation."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    q = _conv_of(p + "q", _project(h, w, p + "q"), w, mem).view(T, H, 2, d)
    if shared is None:
        k = _conv_of(p + "k", _project(h, w, p + "k"), w, mem).view(T, G, 2, d)
        v = _conv_of(p + "v", _project(h, w, p + "v"), w, mem).view(T, G, dv)
        _remember(mem, k, v, positions)
        shared = mem
    lam = differential_lambda(w, p, diff)
    window = int((m.get("mask") or {}).get("size", 0))
    out = h.new_zeros(T, H, dv)
    for head in range(H):
        g = head // (H // G)
        maps = [windowed_softmax_attention(q[:, head, i], shared.k[:, g, i], shared.v[:, g], float(m["scale"]),
                                           positions, shared.pos, window) for i in range(2)]
        out[:, head] = rms_divide(maps[0] - lam * maps[1], eps) * (1.0 - diff)
    return out.reshape(T, H * dv) @ w[p + "o"].T


# ---- feed-forwards ---------------------------------------------------------------------------------
def dense_feed_forward(h, w, p):
    return (F.silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def router_choice(h, w, p, top: int):
    """(chosen experts [T, top], their weights): the softmax over all experts, the largest kept as they are."""
    scores = torch.softmax(h @ w[p + "router"].T, dim=-1)
    weights, chosen = torch.topk(scores, top, dim=-1)
    return chosen, weights


def routed_feed_forward(h, w, p, mlp, forced=None):
    """``forced`` [T, top]: experts to use in place of the router's own choice (their weights stay the router's)."""
    top = int(mlp["router"]["top"])
    chosen, weights = router_choice(h, w, p, top)
    if forced is not None:
        chosen = forced
        weights = torch.softmax(h @ w[p + "router"].T, dim=-1).gather(1, forced)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for c in range(top):
            e = int(chosen[t, c])
            out[t] += weights[t, c] * (torch.relu(h[t] @ w[f"{p}e{e}.up"].T) ** 2 @ w[f"{p}e{e}.down"].T)
    return out


# ---- the model -------------------------------------------------------------------------------------
class SequenceMemory:
    def __init__(self, cfg):
        self.layers = [MixerMemory() for _ in cfg["layers"]]
        self.previous = None
        self.count = 0


def forward(w, cfg, tokens, mem: SequenceMemory | None = None, keep_layers=None, forced=None):
    """Logits [T, vocab] of the next ``tokens`` of one sequence; ``mem`` carries what earlier calls left.
    ``keep_layers``: a list that receives the stream after every layer.  ``forced``: {layer: experts [T, top]}."""
    mem = mem if mem is not None else SequenceMemory(cfg)
    eps, mult = float(cfg["norm"]["eps"]), float(cfg.get("residual_mult", 1.0))
    T = len(tokens)
    positions = torch.arange(mem.count, mem.count + T)
    x = embed(w, cfg, list(tokens), mem.previous)
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = rms_norm(x, w[p + "norm1"], eps)
        src = m.get("kv_from")
        shared = mem.layers[src] if src is not None else None
        if layer["type"] == "attention":
            y = differential_attention(h, w, p + "mix.", m, positions, eps, mem.layers[i], shared)
        elif layer["type"] == "attention_2":
            y = gated_rotary_attention(h, w, p + "mix.", m, positions, mem.layers[i], shared)
        else:
            raise ValueError(layer["type"])
        x = x + mult * rms_norm(y, w[p + "norm1b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = rms_norm(x, w[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                y = dense_feed_forward(h, w, p + "mlp.")
            else:
                y = routed_feed_forward(h, w, p + "mlp.", mlp, None if forced is None else forced.get(i))
            x = x + mult * rms_norm(y, w[p + "norm2b"], eps)
        if keep_layers is not None:
            keep_layers.append(x.clone())
    mem.previous, mem.count = int(tokens[-1]), mem.count + T
    return rms_norm(x, w["final.norm"], eps) @ w["embed"].T
