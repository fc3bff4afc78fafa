"""Dense feed-forwards: SwiGLU, ``down(silu(gate(h)) * up(h))``, and one without gate, ``down(act(up(h)))``;
no biases.

The reference calls the checkpoint's own module for this (tensorline/paged.py:276); the
projection names and shapes are fixed by tensorline/manager.py:52-54 and tensorline/quant.py:25.
Gate and up are fused into one [2I, H] matrix at load; SiLU is computed in float32.
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Linear, Part, TensorGetter, fuse_linears
from tensorline_amd.parts.registry import register_feed_forward


@register_feed_forward("swiglu")
class SwiGLU(Part):
    def __init__(self, hidden_size, prefix, dtype, device, intermediate_size: int, names: tuple | None = None,
                 activation: str = "silu"):
        """``names``: the checkpoint names of the gate, up and down matrices below the prefix where they are
        not ``gate_proj.weight``, ``up_proj.weight`` and ``down_proj.weight``.  ``activation``: what the gate
        passes, "silu" or "gelu_tanh" (the tanh form of GELU), computed in float32."""
        super().__init__(hidden_size, prefix, dtype, device)
        if activation not in kernels.GLU_ACTIVATIONS:
            raise ValueError(f"{prefix}: unknown activation {activation!r}; known: {', '.join(kernels.GLU_ACTIVATIONS)}")
        self.activation = activation
        self.intermediate_size = int(intermediate_size)
        g, u, d = (prefix + n for n in names) if names else (None, None, None)
        self._gate = Linear(prefix + "gate_proj", hidden_size, self.intermediate_size, False, weight_name=g)
        self._up = Linear(prefix + "up_proj", hidden_size, self.intermediate_size, False, weight_name=u)
        self.gate_up: Linear | None = None
        self.down = Linear(prefix + "down_proj", self.intermediate_size, hidden_size, False, weight_name=d)

    def tensors(self):
        return {**self._gate.tensors(), **self._up.tensors(), **self.down.tensors()}

    def load(self, get: TensorGetter) -> None:
        self._gate.load(get)
        self._up.load(get)
        self.gate_up = fuse_linears(self.prefix + "gate_up_proj", [self._gate, self._up])
        self._gate.weight = self._up.weight = None
        self.down.load(get)
        self.down.prepare()

    def weight_tensors(self):
        return self.gate_up.tensors_kept() + self.down.tensors_kept()

    def library_products(self):
        return [(self.gate_up.weight, self.dtype), (self.down.weight, torch.float32)]

    @property
    def defers_norm(self) -> bool:
        # the product that carries a norm has SiLU in its epilogue and no other activation
        return self.activation == "silu" and self.gate_up.shuffled is not None and self.down.shuffled is not None

    keeps_share_sums = True

    def forward(self, h, ctx, sink=None, keep_shares: bool = False):
        if self.activation != "silu":
            act = kernels.swiglu_gate_up(h, self.gate_up.weight, self.gate_up.streamed, activation=self.activation)
            return self.down(act, out_dtype=torch.float32, keep_shares=keep_shares)
        act = kernels.swiglu_gate_up(h, self.gate_up.weight, self.gate_up.streamed)
        return self.down(act, out_dtype=torch.float32, sink=sink, keep_shares=keep_shares)


@register_feed_forward("up_down")
class UpDown(Part):
    """A feed-forward without gate: ``down(act(up(h)))``, no biases.  ``activation``: "relu2", the
    square of relu, computed in float32 (in the product's epilogue in few-row bfloat16 steps, by a pass
    of its own otherwise).  Tensors under the prefix: up, down."""

    ACTIVATIONS = ("relu2",)

    def __init__(self, hidden_size, prefix, dtype, device, ff: int, activation: str = "relu2"):
        super().__init__(hidden_size, prefix, dtype, device)
        if activation not in self.ACTIVATIONS:
            raise ValueError(f"{prefix}: unknown activation {activation!r}; known: {', '.join(self.ACTIVATIONS)}")
        self.ff, self.activation = int(ff), activation
        self.up = Linear(prefix + "up", hidden_size, self.ff, False, weight_name=prefix + "up")
        self.down = Linear(prefix + "down", self.ff, hidden_size, False, weight_name=prefix + "down")

    def tensors(self):
        return {**self.up.tensors(), **self.down.tensors()}

    def load(self, get: TensorGetter) -> None:
        for lin in (self.up, self.down):
            lin.load(get)
            lin.prepare()

    def weight_tensors(self):
        return self.up.tensors_kept() + self.down.tensors_kept()

    def library_products(self):
        return [(self.up.weight, torch.float32), (self.down.weight, torch.float32)]

    def forward(self, h, ctx):
        act = self.up(h, out_dtype=self.dtype, act=self.activation)       # the activation rides on few-row products
        return self.down(act, out_dtype=torch.float32)
