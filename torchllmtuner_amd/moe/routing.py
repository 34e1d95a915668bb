"""Token-choice top-K router on the fused selection kernel.

Constructor surface, validation messages, return contract and hook points of
llmtuner/models/common/moe/routing.py:31-345 (``TokenChoiceTopKRouter``).  The
gate GEMM and the score / top-k / gather / norm / scale chain each run as one
device kernel; ``forward`` returns ``(topk_scores_TK, topk_expert_ids_TK,
routing_map_TE)`` like the reference, ``route`` skips the (T, E) map for callers
that only need ids and weights.

Selection order is "higher choice score first, ties to the lower expert id"; the
reference's ``torch.topk(sorted=False)`` leaves both unspecified.
"""

from __future__ import annotations

import math
from numbers import Real
from typing import Literal

import torch
import torch.nn as nn

from .. import functional as Fn
from .. import ops
from .linear import RouterGateLinear

__all__ = ["TokenChoiceTopKRouter"]


class TokenChoiceTopKRouter(nn.Module):
    def __init__(
        self,
        num_experts: int,
        dim: int,
        top_k: int = 1,
        *,
        score_func: Literal["softmax", "sigmoid", "sqrtsoftplus"] = "sigmoid",
        route_norm: bool = False,
        route_scale: float = 1.0,
        num_expert_groups: int | None = None,
        num_limited_groups: int | None = None,
        aux_loss=None,
        _debug_force_load_balance: bool = False,
        fixed_router: bool = False,
    ) -> None:
        super().__init__()
        for name, value in (
            ("num_experts", num_experts),
            ("dim", dim),
            ("top_k", top_k),
            ("num_expert_groups", num_expert_groups),
            ("num_limited_groups", num_limited_groups),
        ):
            if value is None and name in ("num_expert_groups", "num_limited_groups"):
                continue
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ValueError(f"{name} must be positive integer, got {value!r}")
        if not 1 <= top_k <= num_experts:
            raise ValueError("top_k must be in [1, num_experts]")
        if score_func not in ("sigmoid", "softmax", "sqrtsoftplus"):
            raise ValueError(f"Unknown score function {score_func}")
        if (
            not isinstance(route_scale, Real)
            or isinstance(route_scale, bool)
            or not math.isfinite(route_scale)
        ):
            raise ValueError("route_scale must be a finite real number")
        for name, value in (
            ("fixed_router", fixed_router),
            ("route_norm", route_norm),
            ("_debug_force_load_balance", _debug_force_load_balance),
        ):
            if not isinstance(value, bool):
                raise ValueError(f"{name} must be bool")
        if num_expert_groups is None and num_limited_groups is not None:
            raise ValueError("num_limited_groups requires num_expert_groups")
        if num_expert_groups is not None:
            if num_limited_groups is None:
                raise ValueError("num_limited_groups must be set when num_expert_groups is set")
            if num_limited_groups > num_expert_groups:
                raise ValueError(
                    f"num_limited_groups ({num_limited_groups}) cannot exceed "
                    f"num_expert_groups ({num_expert_groups})"
                )
            if num_experts % num_expert_groups != 0:
                raise ValueError(
                    f"num_experts ({num_experts}) must be divisible by "
                    f"num_expert_groups ({num_expert_groups})"
                )
            if num_experts // num_expert_groups < 2:
                raise ValueError(
                    f"num_experts_per_group ({num_experts // num_expert_groups}) "
                    "must be >= 2 to form a group score"
                )
            if top_k > num_limited_groups * (num_experts // num_expert_groups):
                raise ValueError("top_k exceeds the selected expert groups' capacity")
        self.gate = RouterGateLinear(dim=dim, num_experts=num_experts)
        self.num_experts = num_experts
        self.top_k = top_k
        self.score_func = score_func
        self.route_norm = route_norm
        self.route_scale = route_scale
        self.num_expert_groups = num_expert_groups
        self.num_limited_groups = num_limited_groups
        self.aux_loss = aux_loss
        self._debug_force_load_balance = _debug_force_load_balance
        self.fixed_router = fixed_router

    # -- selection mode of the fused kernel -----------------------------------
    def _mode(self) -> int:
        if self.fixed_router:
            return ops.SELECT_FIXED
        if self._debug_force_load_balance:
            return ops.SELECT_BALANCED
        return ops.SELECT_TOPK

    def _select(self, logits_TE, expert_bias_E, want_scores):
        return Fn.route_select(
            logits_TE,
            expert_bias_E,
            self.top_k,
            self.score_func,
            self.route_norm,
            float(self.route_scale),
            self.num_expert_groups,
            self.num_limited_groups,
            self._mode(),
            want_scores,
        )

    def route(self, x_TD: torch.Tensor, expert_bias_E: torch.Tensor | None = None):
        """Scores and ids only: ``(topk_scores_TK fp32, topk_expert_ids_TK int64)``."""
        logits_TE = self.gate(x_TD)
        scores_TK, ids_TK, _ = self._select(logits_TE, expert_bias_E, False)
        return scores_TK, ids_TK

    def forward(
        self,
        x_TD: torch.Tensor,
        expert_bias_E: torch.Tensor | None = None,
        *,
        padding_mask_T: torch.Tensor | None = None,
    ) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
        if padding_mask_T is not None:
            if padding_mask_T.dtype != torch.bool:
                raise ValueError(f"padding_mask_T must have dtype bool, got {padding_mask_T.dtype}.")
            if padding_mask_T.shape != x_TD.shape[:-1]:
                raise ValueError(
                    "padding_mask_T must have shape matching the routing-map "
                    f"token axis, got {tuple(padding_mask_T.shape)} for scores "
                    f"{(*x_TD.shape[:-1], self.num_experts)}."
                )
        logits_TE = self.gate(x_TD)
        want_scores = self.training and self.aux_loss is not None
        topk_scores_TK, topk_expert_ids_TK, scores_TE = self._select(
            logits_TE, expert_bias_E, want_scores
        )
        # One-hot map of each token's chosen experts; (T, E) bool is index glue, not
        # arithmetic, and is built with a scatter like the reference's.
        routing_map_TE = torch.zeros(
            x_TD.shape[0], self.num_experts, dtype=torch.bool, device=x_TD.device
        ).scatter_(-1, topk_expert_ids_TK, True)

        if want_scores:
            masked_map = (
                routing_map_TE
                if padding_mask_T is None
                else routing_map_TE & ~padding_mask_T.unsqueeze(-1)
            )
            topk_scores_TK = self.aux_loss(
                scores_TE, masked_map, carrier=topk_scores_TK, padding_mask_T=padding_mask_T
            )
        return topk_scores_TK, topk_expert_ids_TK, routing_map_TE
