"""Norms, fused with the residual add that precedes them: RMSNorm and Dynamic Tanh.

``h = forward(x, residual)`` does ``x += residual`` on the float32 residual stream (in place)
and returns ``x / sqrt(mean(x^2) + eps) * weight`` in the activation dtype.  Sum of squares,
scaling and the residual sum are float32 (reference: tensorline/fused.py:19-32,58-69).
"""
from __future__ import annotations

import torch

from tensorline_amd.ops import kernels
from tensorline_amd.parts.base import Part, TensorGetter
from tensorline_amd.parts.registry import register_norm
from tensorline_amd.parts.spec import TensorDecl


@register_norm("rmsnorm")
class RMSNorm(Part):
    def __init__(self, hidden_size, prefix, dtype, device, eps: float, name: str = "weight", around_zero: bool = False):
        """``around_zero``: the checkpoint stores the weight's distance from one, ``x / rms(x) * (1 + w)``; the
        one is added when the weight is loaded (in float32), and every kernel sees a plain weight."""
        super().__init__(hidden_size, prefix, dtype, device)
        self.eps = float(eps)
        self.around_zero = bool(around_zero)
        self.name = prefix + name
        self.weight: torch.Tensor | None = None

    def tensors(self):
        return {self.name: TensorDecl((self.hidden_size,), "normal" if self.around_zero else "one_plus_normal", 0.1, "float32")}

    def load(self, get: TensorGetter) -> None:
        self.weight = get(self.name)
        if self.around_zero:
            self.weight = (self.weight.to(torch.float32) + 1.0).contiguous()

    def weight_tensors(self):
        return [self.weight]

    adds_share_sums = True
    adds_normed_branch = True      # ``forward`` takes a kernels.NormedBranch as the residual

    def as_branch(self, y: torch.Tensor, mult: float) -> "kernels.NormedBranch":
        """``mult * norm(y)``, left for the norm that reads the stream next to add in its own pass."""
        return kernels.NormedBranch(y, self.weight, self.eps, float(mult))

    def deferrable(self) -> tuple[torch.Tensor, float]:
        """(weight, eps): all a product needs to carry this norm (see ``Part.defers_norm``)."""
        return self.weight, self.eps

    def forward(self, x: torch.Tensor, residual=None, rows: torch.Tensor | None = None) -> torch.Tensor:
        return kernels.add_rmsnorm(x, residual, self.weight, self.eps, self.dtype, rows=rows)


@register_norm("dyt")
class DynamicTanh(Part):
    """Dynamic Tanh in the place of a norm: ``tanh(alpha * x) * weight + bias`` with a learned scalar
    ``alpha``; no mean or variance of the row is taken.  Tensors: ``name`` (weight), ``name + ".b"``,
    ``name + ".alpha"`` (a scalar).  Same interface as the RMS norm: adds ``residual`` into the float32
    stream first, in place, or works on ``rows`` only.  It cannot be carried by the products around
    it (it is not one factor per row), so it offers no ``deferrable``."""

    def __init__(self, hidden_size, prefix, dtype, device, name: str):
        super().__init__(hidden_size, prefix, dtype, device)
        self.name = prefix + name
        self.weight = self.bias = self.alpha = None

    def tensors(self):
        return {self.name: TensorDecl((self.hidden_size,), "one_plus_normal", 0.1, "float32"),
                self.name + ".b": TensorDecl((self.hidden_size,), "normal", 0.1, "float32"),
                self.name + ".alpha": TensorDecl((), "one_plus_normal", 0.2, "float32")}

    def load(self, get: TensorGetter) -> None:
        self.weight, self.bias = get(self.name), get(self.name + ".b")
        self.alpha = get(self.name + ".alpha").reshape(1).contiguous()

    def weight_tensors(self):
        return [self.weight, self.bias, self.alpha]

    def forward(self, x: torch.Tensor, residual=None, rows: torch.Tensor | None = None) -> torch.Tensor:
        return kernels.add_dyt(x, residual, self.weight, self.bias, self.alpha, self.dtype, rows=rows)
