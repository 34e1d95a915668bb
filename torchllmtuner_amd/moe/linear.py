"""The router's projection: one score per expert, always in fp32.

Interface of llmtuner/models/common/linear.py:154-183 (``RouterGateLinear``): an
``nn.Linear`` subclass with ``weight (E, D)`` and a ``bias`` attribute that exists
(as ``None``) when built without one; forward and backward GEMMs run in fp32 on
the device kernels whatever the storage dtype.
"""

from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops as Fn

__all__ = ["RouterGateLinear"]


class RouterGateLinear(nn.Linear):
    def __init__(self, dim: int, num_experts: int, *, bias: bool = False) -> None:
        super().__init__(dim, num_experts, bias=bias)

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        lead = input.shape[:-1]
        x = input.reshape(-1, input.shape[-1]) if input.dim() != 2 else input
        out = Fn.router_gate(x, self.weight, self.bias)
        return out.reshape(*lead, out.shape[-1]) if input.dim() != 2 else out
