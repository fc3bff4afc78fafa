"""Routed experts: a feed-forward of many small gated layers of which every token uses a few.

    z = W_router h + b  (float32);  the ``top`` experts with the largest z, weights = softmax over
    those ``top`` logits alone;  out = sum_chosen weight_e * expert_e(h)  (+ shared(h))
    expert(h) = W_down (g * sigmoid(alpha g) * (u + 1)),  g = min(W_gate h, limit),  u = clamp(W_up h, +-limit)

Other designs change the weights (``weighting`` "sigmoid": each chosen expert by its own score,
``router_scale * sigmoid(z_e)``, not renormalised; "softmax_all": the chosen experts' shares of the
softmax over all experts, not renormalised), leave the router without bias, use the plain gated
activation ``silu(g) * u`` (``activation`` "swiglu": no limit, alpha 1, nothing added to u), or have
experts without gate, ``W_down relu(W_up h)^2`` (``activation`` "relu2": tensors e<i>.up / .down only).
``weighting`` "sigmoid_grouped": scores are ``sigmoid(z)``; the experts form ``groups`` equal groups of neighbours, a
group's score is the sum of its two largest scores, only experts of the ``keep_groups`` best groups can be chosen,
and the chosen experts' weights are their scores divided by their sum.  A shared expert has the experts' activation
(its ``limit`` only with the clamped one) and, with ``shared`` = {ff, gate: True}, is multiplied by
``sigmoid(W_sg h)``, one number per token (``shared.sg`` [1, width]), before it is added.

The experts' matrices are stacked ([experts, 2 ff, width] gate over up, [experts, width, ff]); a
step's (token, choice) pairs are ordered by expert on the device and both products run as one
grouped launch each (``kernels.moe_experts``), with no look at the device from the host, so the
step can be captured in a graph.  The shared expert, which every token uses, is a plain dense
feed-forward of the same form on the framework's ordinary products.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_feed_forward
from tensorline_amd.parts.spec import TensorDecl


@register_feed_forward("routed_experts")
class RoutedExperts(Part):
    """Parameters: ``experts``, ``top``, ``ff`` and ``limit`` of an expert, ``shared`` = {ff, limit} or
    None, ``alpha`` of the gate's sigmoid; ``weighting`` ("softmax_top", "sigmoid" or "softmax_all"),
    ``router_scale``, ``router_bias``, ``activation`` ("clamped_glu", "swiglu" or "relu2"), ``groups`` and ``keep_groups``
    (with the weighting "sigmoid_grouped").  Tensors under the prefix: router,
    router.b, e<i>.gate / .up / .down, shared.gate / .up / .down / .sg."""

    def __init__(self, hidden_size, prefix, dtype, device, experts: int, top: int, ff: int, limit: float | None = None,
                 shared: dict | None = None, alpha: float = 1.702, weighting: str = "softmax_top", router_scale: float = 1.0,
                 router_bias: bool = True, activation: str = "clamped_glu", groups: int = 1, keep_groups: int | None = None):
        super().__init__(hidden_size, prefix, dtype, device)
        if activation not in ("clamped_glu", "swiglu", "relu2") or weighting not in kernels.ROUTER_WEIGHTINGS:
            raise ValueError(f"{prefix}: unknown activation {activation!r} or weighting {weighting!r}")
        self.gated = activation != "relu2"
        if activation in ("swiglu", "relu2"):
            limit, alpha, self.shift = float("inf"), 1.0, 0.0
        else:
            if limit is None:
                raise ValueError(f"{prefix}: the clamped activation needs its limit")
            self.shift = 1.0
        if shared and activation == "relu2":
            raise ValueError(f"{prefix}: a shared expert comes with a gated activation only")
        self.activation = activation
        self.weighting, self.router_scale = weighting, float(router_scale)
        self.groups = int(groups)
        self.keep_groups = self.groups if keep_groups is None else int(keep_groups)
        if self.groups <= 0 or int(experts) % self.groups or not 0 < self.keep_groups <= self.groups or self.groups > 64:
            raise ValueError(f"{prefix}: {experts} experts do not form {groups} equal groups (at most 64) of which {keep_groups} are kept")
        if self.groups > 1 and weighting != "sigmoid_grouped":
            raise ValueError(f"{prefix}: groups of experts come with the weighting 'sigmoid_grouped'")
        if int(top) > self.keep_groups * (int(experts) // self.groups):
            raise ValueError(f"{prefix}: {top} choices are more than the {self.keep_groups} kept groups hold")
        self.experts, self.top, self.ff, self.limit, self.alpha = int(experts), int(top), int(ff), float(limit), float(alpha)
        if not 0 < self.top <= self.experts or self.top > 32 or self.experts > 1024:
            raise ValueError(f"{prefix}: top {self.top} of {self.experts} experts is not served (top <= 32, experts <= 1024)")
        self.router = Linear(prefix + "router", hidden_size, self.experts, bool(router_bias), weight_name=prefix + "router",
                             bias_name=prefix + "router.b")
        self.gate_up = self.down = None
        self.shared_ff = int(shared["ff"]) if shared else 0
        self.shared_limit = float(shared.get("limit", float("inf"))) if shared else 0.0
        self.shared_gated = bool(shared and shared.get("gate"))      # the shared expert times sigmoid(W_sg h), per token
        self._sg = self._su = self.shared_gate_up = self.shared_down = None
        if shared:
            p = prefix + "shared."
            self._sg = Linear(p + "gate", hidden_size, self.shared_ff, False, weight_name=p + "gate")
            self._su = Linear(p + "up", hidden_size, self.shared_ff, False, weight_name=p + "up")
            self.shared_down = Linear(p + "down", self.shared_ff, hidden_size, False, weight_name=p + "down")
        self._token_gate = Linear(prefix + "shared.sg", hidden_size, 1, False, weight_name=prefix + "shared.sg") \
            if self.shared_gated else None

    def tensors(self):
        out = dict(self.router.tensors())
        if self._token_gate is not None:
            out.update(self._token_gate.tensors())
        for e in range(self.experts):
            p = f"{self.prefix}e{e}."
            if self.gated:
                out[p + "gate"] = TensorDecl((self.ff, self.hidden_size), "normal", 0.05, "compute")
            out[p + "up"] = TensorDecl((self.ff, self.hidden_size), "normal", 0.05, "compute")
            out[p + "down"] = TensorDecl((self.hidden_size, self.ff), "normal", 0.05, "compute")
        if self.shared_down is not None:
            for lin in (self._sg, self._su, self.shared_down):
                out.update(lin.tensors())
        return out

    def load(self, get: TensorGetter) -> None:
        self.router.load(get)
        if self._token_gate is not None:
            # the gate's one row rides on the router's product: logits [T, experts | gate]
            self._token_gate.load(get)
            self.router = fuse_linears(self.prefix + "router_sg", [self.router, self._token_gate])
            self._token_gate.weight = None
        else:
            self.router.prepare()
        name = lambda e, s: f"{self.prefix}e{e}.{s}"
        if self.gated:
            self.gate_up = torch.stack([torch.cat([get(name(e, "gate")), get(name(e, "up"))]) for e in range(self.experts)]).contiguous()
        else:
            self.gate_up = torch.stack([get(name(e, "up")) for e in range(self.experts)]).contiguous()
        self.down = torch.stack([get(name(e, "down")) for e in range(self.experts)]).contiguous()
        if self.shared_down is not None:
            self._sg.load(get)
            self._su.load(get)
            self.shared_gate_up = fuse_linears(self.prefix + "shared.gate_up", [self._sg, self._su])
            self._sg.weight = self._su.weight = None
            self.shared_down.load(get)
            self.shared_down.prepare()

    def weight_tensors(self):
        out = self.router.tensors_kept() + [self.gate_up, self.down]
        if self.shared_down is not None:
            out += self.shared_gate_up.tensors_kept() + self.shared_down.tensors_kept()
        return out

    def library_products(self):
        if self.shared_down is None:
            return []
        return [(self.shared_gate_up.weight, self.dtype), (self.shared_down.weight, torch.float32)]

    def forward(self, h, ctx):
        logits = self.router(h, out_dtype=torch.float32)
        ids, weights = kernels.moe_route(logits, self.top, self.weighting, self.router_scale, experts=self.experts,
                                         groups=self.groups, keep=self.keep_groups)
        shared = None
        if self.shared_down is not None:
            if self.activation == "swiglu":       # SiLU rides on the few-row product, as in the dense feed-forward
                act = kernels.swiglu_gate_up(h, self.shared_gate_up.weight, self.shared_gate_up.streamed)
            else:
                act = kernels.clamp_glu(self.shared_gate_up(h, out_dtype=torch.float32), self.shared_limit, self.alpha, self.dtype)
            shared = self.shared_down(act, out_dtype=torch.float32)
        token_gate = logits[:, self.experts:self.experts + 1] if self.shared_gated else None     # applied where it is added
        return kernels.moe_experts(h, self.gate_up, self.down, ids, weights, self.limit, self.alpha, shared, self.shift,
                                   gated=self.gated, shared_gate=token_gate)
