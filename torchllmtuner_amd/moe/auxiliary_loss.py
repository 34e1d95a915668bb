"""Auxiliary-loss gradient injection and the per-forward load-balance loss.

Mirrors ``llmtuner/models/common/aux_loss.py`` (``AuxLoss``: coefficient, step
denominator, identity-forward injection, per-instance metric accumulator) and
``llmtuner/models/common/moe/auxiliary_loss.py`` (``MicrobatchWiseLoadBalanceLoss``) for
one process: the token axis is not sharded here, so the reference's token-partition
all-reduce is the identity.  The loss arithmetic and its gradient run in the HIP kernels
behind ``ops.balance_loss_fwd / balance_loss_bwd``.
"""

from __future__ import annotations

import re
from collections import defaultdict
from collections.abc import Sequence
from contextvars import ContextVar
from typing import ClassVar

import torch
import torch.nn as nn
from torch.autograd.function import once_differentiable

from .. import ops

__all__ = ["AuxLoss", "AuxLossInjection", "MicrobatchWiseLoadBalanceLoss", "in_checkpoint_recompute"]

# Activation-checkpoint replays set this so metric side effects are not counted twice
# (aux_loss.py:39-44); the injection itself stays in the graph.
in_checkpoint_recompute: ContextVar[bool] = ContextVar("in_checkpoint_recompute", default=False)


class AuxLossInjection(torch.autograd.Function):
    """Identity on ``carrier``; the backward hands the loss a gradient of one
    (aux_loss.py:72-90: coefficient and 1/denominator are already folded into the value)."""

    @staticmethod
    def forward(ctx, carrier, aux_loss):
        ctx.save_for_backward(aux_loss)
        return carrier

    @staticmethod
    def backward(ctx, grad_carrier):
        (aux_loss,) = ctx.saved_tensors
        return grad_carrier, torch.ones_like(aux_loss)


class AuxLoss(nn.Module):
    """Base class: subclasses call ``inject()`` each forward (aux_loss.py:93-238)."""

    _group_counts: ClassVar[dict[tuple[str, str], int]] = defaultdict(int)
    _step_denominator: ClassVar[torch.Tensor | None] = None

    def __init__(self, *, coeff: float, reduce_mesh: str = "batch") -> None:
        super().__init__()
        self.coeff = coeff
        self.reduce_mesh = reduce_mesh
        self._runtime_denominator: torch.Tensor | None = None
        self.register_buffer("instance_acc", torch.zeros((), dtype=torch.float32), persistent=False)
        AuxLoss._group_counts[(self.reduce_mesh, self.metric_name)] += 1

    @property
    def metric_name(self) -> str:
        return re.sub(r"(?<=[a-z])(?=[A-Z])|(?<=[A-Z])(?=[A-Z][a-z])", "_", type(self).__name__).lower()

    @classmethod
    def set_step_denominator(cls, denominator: torch.Tensor, *,
                             model_parts: Sequence[nn.Module] | None = None) -> None:
        """The step's global routed-token count, set before the first forward."""
        if model_parts is None:
            cls._step_denominator = denominator
            return
        seen: set[int] = set()
        for part in model_parts:
            for module in part.modules():
                if isinstance(module, AuxLoss) and id(module) not in seen:
                    seen.add(id(module))
                    module._runtime_denominator = denominator
                    module.instance_acc.zero_()

    def inject(self, raw_sum: torch.Tensor, *, carrier: torch.Tensor) -> torch.Tensor:
        denominator = self._runtime_denominator
        if denominator is None:
            denominator = AuxLoss._step_denominator
        if denominator is None:
            raise ValueError(
                "AuxLoss.set_step_denominator() must be called with the "
                "step's global routed-token count before the first forward."
            )
        # clamp_min(1): an all-padding step has zero routed tokens
        scale = 1.0 / denominator.to(raw_sum.device).clamp_min(1)
        injected = raw_sum * (self.coeff * scale)
        with torch.no_grad():
            if not in_checkpoint_recompute.get():
                self.instance_acc.add_((raw_sum * scale).detach().to(self.instance_acc.device))
        return AuxLossInjection.apply(carrier, injected)


class MicrobatchWiseLoadBalanceLoss(AuxLoss):
    """``sum_i f_i p_i`` over one forward's tokens (auxiliary_loss.py:30-168):
    ``f_i = E * counts_i / sum_j counts_j``, ``p_i = sum_t s_ti / sum_j s_tj``."""

    def __init__(self, *, coeff: float, token_replication_size: int = 1) -> None:
        if (not isinstance(token_replication_size, int) or isinstance(token_replication_size, bool)
                or token_replication_size < 1):
            raise ValueError("token_replication_size must be a positive integer")
        super().__init__(coeff=coeff, reduce_mesh="batch")
        self.token_replication_size = token_replication_size

    def _reduce_token_partials(self, partial_E: torch.Tensor, axes: tuple[str, ...]) -> torch.Tensor:
        """No mesh axis shards the token stream in a single process: the identity."""
        return partial_E

    def forward(self, scores_TE: torch.Tensor, routing_map_TE: torch.Tensor, *, carrier: torch.Tensor,
                padding_mask_T: torch.Tensor | None = None) -> torch.Tensor:
        loss, _f_E = ops.balance_loss_fwd(scores_TE, routing_map_TE, padding_mask_T)
        if self.token_replication_size > 1:
            loss = loss.detach() + (loss - loss.detach()) / self.token_replication_size
        return self.inject(loss, carrier=carrier)
