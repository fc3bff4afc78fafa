"""A plain, slow implementation of the Kabulix decoder, one function per mechanism, in float64 on the CPU.

It shares no code with the product.  ``weights`` maps tensor names to tensors; ``config`` is the dictionary of
``config.json``.  A whole sequence is computed at once with explicit loops over queries and keys, so nothing here
knows of pages, steps or batches.

Notation: ``h`` [T, width] is a mixer's or feed-forward's input, ``pos`` the tokens' positions 0..T-1.
"""
from __future__ import annotations

import math

import torch

F = torch.float64


# ---- small pieces -------------------------------------------------------------------------------
def rms_scale(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, w, eps):
    """RMS norm whose stored weight is the distance from one."""
    return rms_scale(x, eps) * (1.0 + w)


def norm_plain(x, w, eps):
    return rms_scale(x, eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def frequencies(dims: int, base: float, scaling: dict | None) -> tuple[list[float], float]:
    """(f_i for i < dims / 2, the factor on cosine and sine)."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def turn_dim(turns):
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(turn_dim(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn_dim(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1.0 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def turn_pairs(x: torch.Tensor, pos, freqs, mag: float) -> torch.Tensor:
    """x [T, ..., n]: neighbours (2i, 2i + 1) of the first 2 len(freqs) entries are turned by pos * f_i."""
    out = x.clone()
    for t in range(x.shape[0]):
        for i, f in enumerate(freqs):
            a = float(pos[t]) * f
            c, s = math.cos(a) * mag, math.sin(a) * mag
            u, v = x[t, ..., 2 * i], x[t, ..., 2 * i + 1]
            out[t, ..., 2 * i] = u * c - v * s
            out[t, ..., 2 * i + 1] = v * c + u * s
    return out


# ---- who sees whom --------------------------------------------------------------------------------
def sees_window_and_first(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def sees_window(i: int, j: int, size: int) -> bool:
    return 0 <= i - j < size


def sees_chunk(i: int, j: int, size: int) -> bool:
    return j <= i and i // size == j // size


def sight(pos, sees) -> torch.Tensor:
    """[T, T] of booleans: whether the token in row i sees the token in column j."""
    T = len(pos)
    return torch.tensor([[sees(int(pos[i]), int(pos[j])) for j in range(T)] for i in range(T)])


def softmax_attention(q, k, v, mask, scale: float) -> torch.Tensor:
    """q [T, dk], k [T, dk], v [T, dv] of one head: row i is the softmax-weighted mean of the v_j it sees."""
    s = (q @ k.T) * scale
    w = torch.softmax(s.masked_fill(~mask, float("-inf")), dim=1)
    return w @ v


# ---- mixers ---------------------------------------------------------------------------------------
def mixer_attention(h, pos, W, p: str, m: dict, eps: float) -> torch.Tensor:
    """Grouped heads, biased q and k, values = the keys as projected, q/k norm per head, partial rotation,
    window plus the first tokens."""
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = k.clone()
    q = norm_plain(q, W[p + "q.norm"], eps)
    k = norm_plain(k, W[p + "k.norm"], eps)
    if m.get("rot"):
        freqs, mag = frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
        q, k = turn_pairs(q, pos, freqs, mag), turn_pairs(k, pos, freqs, mag)
    mask = m.get("mask")
    sees = (lambda i, j: sees_window_and_first(i, j, mask["size"], mask.get("keep_first", 0))) if mask else (lambda i, j: j <= i)
    seen = sight(pos, sees)
    heads = [softmax_attention(q[:, a], k[:, a // (H // G)], v[:, a // (H // G)], seen, m["scale"]) for a in range(H)]
    return torch.cat(heads, 1) @ W[p + "o"].T


def mixer_latent(h, pos, W, p: str, m: dict, eps: float) -> torch.Tensor:
    """Keys and values rebuilt from one normed latent per token; one turned key part for all heads; a gate per
    output column."""
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, d + dr)
    down = h @ W[p + "dkv"].T
    c = norm_plain(down[:, :r], W[p + "dkv.norm"], eps)
    freqs, mag = frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"].get("scaling"))
    k_turned = turn_pairs(down[:, r:], pos, freqs, mag)
    q_turned = turn_pairs(q[:, :, d:], pos, freqs, mag)
    k_plain = (c @ W[p + "uk"].T).view(T, H, d)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    mask = m.get("mask")
    sees = (lambda i, j: sees_window(i, j, mask["size"])) if mask else (lambda i, j: j <= i)
    heads, seen = [], sight(pos, sees)
    for a in range(H):
        qa = torch.cat([q[:, a, :d], q_turned[:, a]], 1)
        ka = torch.cat([k_plain[:, a], k_turned], 1)
        heads.append(softmax_attention(qa, ka, v[:, a], seen, m["scale"]))
    o = torch.cat(heads, 1) * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


def mixer_chunked(h, pos, W, p: str, m: dict) -> torch.Tensor:
    """Grouped heads without positions; a token sees its own chunk of positions up to itself; a gate per head."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, d)
    k = (h @ W[p + "k"].T).view(T, G, d)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    mask = m.get("mask")
    sees = (lambda i, j: sees_chunk(i, j, mask["size"])) if mask else (lambda i, j: j <= i)
    gate = torch.sigmoid(h @ W[p + "g"].T)                   # [T, H]
    seen = sight(pos, sees)
    heads = [softmax_attention(q[:, a], k[:, a // (H // G)], v[:, a // (H // G)], seen, m["scale"]) * gate[:, a:a + 1]
             for a in range(H)]
    return torch.cat(heads, 1) @ W[p + "o"].T


# ---- feed-forwards --------------------------------------------------------------------------------
def gated_ff(h, W, p: str, act) -> torch.Tensor:
    return (act(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(z: torch.Tensor, top: int, groups: int, keep: int) -> tuple[list[int], list[float]]:
    """One token's router logits -> (chosen experts, their weights)."""
    s = torch.sigmoid(z)
    E = s.shape[0]
    per = E // groups
    group_score = []
    for g in range(groups):
        part = sorted((float(x) for x in s[g * per:(g + 1) * per]), reverse=True)
        group_score.append(sum(part[:2]))
    kept = sorted(range(groups), key=lambda g: (-group_score[g], g))[:keep]
    allowed = [e for e in range(E) if e // per in kept]
    chosen = sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]
    total = sum(float(s[e]) for e in chosen) + 1e-20
    return chosen, [float(s[e]) / total for e in chosen]


def ff_experts(h, W, p: str, mlp: dict, forced=None, seen=None) -> torch.Tensor:
    """``forced``: per token the experts to use instead of the router's own choice (their weights still come from
    the scores).  ``seen``: a list that gets the router's logits [T, experts]."""
    r = mlp["router"]
    groups = (r.get("groups") or {}).get("count", 1)
    keep = (r.get("groups") or {}).get("keep", groups)
    out = torch.zeros_like(h)
    z = h @ W[p + "router"].T
    if seen is not None:
        seen.append(z.clone())
    for t in range(h.shape[0]):
        chosen, weights = route(z[t], r["top"], groups, keep)
        if forced is not None:
            chosen = [int(e) for e in forced[t]]
            s = torch.sigmoid(z[t])
            total = sum(float(s[e]) for e in chosen) + 1e-20
            weights = [float(s[e]) / total for e in chosen]
        for e, w in zip(chosen, weights):
            out[t] += w * gated_ff(h[t:t + 1], W, f"{p}e{e}.", silu)[0]
    if mlp.get("shared"):
        out = out + gated_ff(h, W, p + "shared.", silu) * torch.sigmoid(h @ W[p + "shared.sg"].T)
    return out


def is_close_call(z: torch.Tensor, taken, mlp: dict, slack: float) -> bool:
    """Whether the experts ``taken`` are what the router chooses once every logit may move by up to ``slack``: tried
    with theirs up and the others down, with one group at a time down and everything else up (a close call between
    two groups neither of which holds a chosen expert), and with a few hundred random moves."""
    r = mlp["router"]
    groups = (r.get("groups") or {}).get("count", 1)
    keep = (r.get("groups") or {}).get("keep", groups)
    want = sorted(int(e) for e in taken)
    E = z.shape[0]
    per = E // groups
    moves = [torch.full((E,), -slack, dtype=F)]
    for e in want:
        moves[0][e] = slack
    for g in range(groups):
        m = torch.full((E,), slack, dtype=F)
        m[g * per:(g + 1) * per] = -slack
        moves.append(m)
        moves.append(torch.where(moves[0] > 0, moves[0], m))
    gen = torch.Generator().manual_seed(0)
    moves += [(torch.rand(E, generator=gen, dtype=F) * 2 - 1) * slack for _ in range(300)]
    return any(sorted(route(z + m, r["top"], groups, keep)[0]) == want for m in moves)


def mixer(kind: str, h, pos, W, p: str, m: dict, eps: float) -> torch.Tensor:
    if kind == "attention":
        return mixer_attention(h, pos, W, p, m, eps)
    if kind == "latent_attention":
        return mixer_latent(h, pos, W, p, m, eps)
    if kind == "attention_2":
        return mixer_chunked(h, pos, W, p, m)
    raise ValueError(kind)


def as_double(weights: dict) -> dict:
    return {k: v.to(F) for k, v in weights.items() if v.dtype.is_floating_point}


# ---- the model ------------------------------------------------------------------------------------
def forward(config: dict, weights: dict, tokens, forced_experts=None, want_layers: bool = False, router_logits=None):
    """Logits [T, vocab] of one sequence from position 0 (and the stream after every layer, if asked).
    ``forced_experts``: {layer index: per token the experts to use}; ``router_logits``: a dictionary that gets
    {layer index: the router's logits [T, experts]}."""
    W = as_double(weights)
    eps = config["norm"]["eps"]
    T = len(tokens)
    pos = list(range(T))
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)]
    after = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}."
        h = norm_around_zero(x, W[p + "norm1"], eps)
        x = x + mixer(layer["type"], h, pos, W, p + "mix.", layer["mixer"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = norm_around_zero(x, W[p + "norm2"], eps)
            if mlp["kind"] == "dense":
                x = x + gated_ff(h, W, p + "mlp.", gelu_tanh)
            else:
                seen = [] if router_logits is not None else None
                x = x + ff_experts(h, W, p + "mlp.", mlp, None if forced_experts is None else forced_experts.get(i), seen)
                if seen:
                    router_logits[i] = seen[0]
        after.append(x.clone())
    logits = norm_around_zero(x, W["final.norm"], eps) @ W["embed"].T
    return (logits, torch.stack(after)) if want_layers else logits
