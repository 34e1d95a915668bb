"""Gated activation marker modules (llmtuner/models/common/activation.py:20-37).

The grouped expert kernels fuse ``silu(gate) * up`` into the gate/up GEMM epilogue,
so ``SwiGLU`` is the only activation the device path accepts; the module is kept
so the constructor surface (``activation_fn=``) matches the reference.
"""

from __future__ import annotations

from abc import ABC, abstractmethod

import torch
import torch.nn as nn
import torch.nn.functional as F

__all__ = ["ActivationFn", "SwiGLU"]


class ActivationFn(nn.Module, ABC):
    @abstractmethod
    def forward(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        raise NotImplementedError


class SwiGLU(ActivationFn):
    """``silu(gate) * up``; evaluated inside the gate/up kernel on the device path."""

    def forward(self, gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
        return F.silu(gate) * up
