"""Gated activations of the expert MLP (llmtuner/models/common/activation.py:20-64).

``SwiGLU`` is fused into the gate/up kernel's epilogue on the device path.  Any other
``ActivationFn`` -- ``SituGLU`` here, or a caller's own module -- runs between three grouped
linear maps (``ops.grouped_linear``): gate and up projections, the module's own torch
arithmetic and autograd, the down projection.
"""

from __future__ import annotations

import math
from abc import ABC, abstractmethod

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["ActivationFn", "SwiGLU", "SituGLU"]


def _soft_clip(x: torch.Tensor, limit: float) -> torch.Tensor:
    """``limit * tanh(x / limit)``: the identity near zero, saturating at +-limit."""
    return torch.tanh(x / limit) * limit


def _require(ok: bool, message: str) -> None:
    if not ok:
        raise ValueError(message)


class ActivationFn(nn.Module, ABC):
    """A gated activation: ``(gate, up)`` of one shape in, one tensor of that shape out."""

    @abstractmethod
    def forward(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class SwiGLU(ActivationFn):
    """``silu(gate) * up``.  The grouped experts evaluate it inside their gate/up kernel and never
    call this method; it serves callers that use the module on its own."""

    def forward(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return F.silu(gate) * up


class SituGLU(ActivationFn):
    """The bounded gate of the Kimi models (llmtuner/models/common/activation.py:40-64):

        ``soft_clip(gate, beta) * sigmoid(gate) * up``,

    with ``up`` itself soft-clipped to ``linear_beta`` when that is given and nonzero.  The
    arithmetic is fp32 whatever the inputs are; the result has the gate's dtype.  Constructor
    checks and their messages are the reference's.
    """

    def __init__(self, beta: float = 1.0, linear_beta: float | None = None) -> None:
        super().__init__()
        _require(math.isfinite(beta) and beta > 0, "SituGLU beta must be finite and positive")
        _require(linear_beta is None or (math.isfinite(linear_beta) and linear_beta >= 0),
                 "SituGLU linear_beta must be finite and nonnegative")
        self.beta = beta
        self.linear_beta = linear_beta

    def _clips_up(self) -> bool:
        return self.linear_beta is not None and self.linear_beta != 0.0

    def forward(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        g32, u32 = gate.to(torch.float32), up.to(torch.float32)
        if self._clips_up():
            u32 = _soft_clip(u32, self.linear_beta)
        out = _soft_clip(g32, self.beta) * torch.sigmoid(g32) * u32
        return out.to(gate.dtype)

    def extra_repr(self) -> str:
        return f"beta={self.beta}, linear_beta={self.linear_beta}"
