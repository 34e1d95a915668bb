"""Token-choice top-K router on the fused selection kernel.

Constructor surface, validation messages, return contract and hook points of
llmtuner/models/common/moe/routing.py:31-345 (``TokenChoiceTopKRouter``).  The
gate GEMM and the score / top-k / gather / norm / scale chain each run as one
device kernel; ``forward`` returns ``(topk_scores_TK, topk_expert_ids_TK,
routing_map_TE)`` like the reference (the select kernel writes the bool map itself);
``route`` skips the (T, E) map for callers that only need ids and weights.

Selection order is "higher choice score first, ties to the lower expert id"; the
reference's ``torch.topk(sorted=False)`` leaves both unspecified.
"""

from __future__ import annotations

import math
from numbers import Real
from typing import Literal

import torch
import torch.nn as nn

from .. import ops as Fn
from .. import ops
from .auxiliary_loss import in_checkpoint_recompute
from .linear import RouterGateLinear

__all__ = ["QuantileBalancedTopKRouter", "QuantileBalancer", "TokenChoiceTopKRouter"]


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

    def _select(self, logits_TE, expert_bias_E, want_scores, padding_mask_T=None, want_map=False):
        """``(scores_TK, ids_TK, scores_TE or None, routing_map_TE or None)``."""
        # padding_mask_T is for subclasses that keep statistics (the quantile router)
        out = Fn.route_select(
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
            want_map,
        )
        return out if want_map else (*out, None)

    def route(self, x_TD: torch.Tensor, expert_bias_E: torch.Tensor | None = None, *,
              padding_mask_T: torch.Tensor | None = None):
        """Scores and ids only: ``(topk_scores_TK fp32, topk_expert_ids_TK int64)``.
        ``padding_mask_T`` only matters to routers that keep statistics."""
        logits_TE = self.gate(x_TD)
        scores_TK, ids_TK, _, _ = self._select(logits_TE, expert_bias_E, False)
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
        topk_scores_TK, topk_expert_ids_TK, scores_TE, routing_map_TE = self._select(
            logits_TE, expert_bias_E, want_scores, padding_mask_T, want_map=True
        )
        if routing_map_TE is None:
            # a selection path without the map output: the reference's scatter (index glue)
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


class QuantileBalancer(nn.Module):
    """Required-bias histogram of quantile-balanced routing and the bias read back from it
    (llmtuner/models/common/moe/routing.py:491-610).

    For sigmoid scores in [0, 1] the bias an expert needs to win a token lies between the
    smallest current bias minus one and the largest plus one; every training micro-batch
    adds ``cutoff - score`` of each (token, expert) pair to ``num_bins`` uniform bins over
    that interval (one device kernel, int64 counters), and ``estimate_expert_bias`` reads
    the ``top_k / num_experts`` quantile of every expert back out (one device kernel).
    The histogram is scratch state: it follows device moves and never lands in a checkpoint.
    """

    def __init__(self, num_experts: int, top_k: int, num_bins: int) -> None:
        super().__init__()
        for name, value in (("num_experts", num_experts), ("top_k", top_k), ("num_bins", num_bins)):
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ValueError(f"{name} must be positive integer, got {value!r}")
        if not 0 < top_k < num_experts:
            raise ValueError(f"top_k ({top_k}) must be between zero and num_experts ({num_experts})")
        self.num_experts = num_experts
        self.top_k = top_k
        self.num_bins = num_bins
        self.register_buffer(
            "required_bias_histogram_EB",
            torch.zeros(num_experts, num_bins, dtype=torch.int64),
            persistent=False,
        )

    @torch.no_grad()
    def observe(self, scores_TE, cutoff_T1, expert_bias_E, *, padding_mask_T=None) -> None:
        """Accumulate one micro-batch; padding tokens and checkpoint replays are skipped."""
        if not self.training or in_checkpoint_recompute.get():
            return
        ops.quantile_observe(
            self.required_bias_histogram_EB, scores_TE, cutoff_T1, expert_bias_E, padding_mask_T
        )

    @torch.no_grad()
    def estimate_expert_bias(self, histogram_EB, expert_bias_E):
        """The next mean-centred bias; an empty histogram returns a copy of the current one."""
        if histogram_EB.shape != (self.num_experts, self.num_bins):
            raise ValueError(
                f"histogram_EB must have shape {(self.num_experts, self.num_bins)}, "
                f"got {tuple(histogram_EB.shape)}"
            )
        return ops.quantile_estimate(histogram_EB, expert_bias_E, self.top_k)


class QuantileBalancedTopKRouter(TokenChoiceTopKRouter):
    """Top-k router balanced by a histogram-estimated quantile bias
    (llmtuner/models/common/moe/routing.py:348-430).

    A training forward takes one biased top-(K+1): the first K experts route the token,
    the (K+1)-th biased score is the cutoff the required biases are measured against.
    Sigmoid scores only, no group-limited routing, no debug routings -- as in the
    reference, whose constructor takes none of those arguments.  Eval routes with the
    plain biased top-k and observes nothing.
    """

    def __init__(
        self,
        num_experts: int,
        dim: int,
        top_k: int = 1,
        *,
        num_bins: int = 1000,
        route_norm: bool = False,
        route_scale: float = 1.0,
        aux_loss=None,
    ) -> None:
        super().__init__(
            num_experts=num_experts, dim=dim, top_k=top_k, score_func="sigmoid",
            route_norm=route_norm, route_scale=route_scale, aux_loss=aux_loss,
        )
        self.quantile_balancer = QuantileBalancer(num_experts=num_experts, top_k=top_k, num_bins=num_bins)

    def _require_bias(self, expert_bias_E):
        if expert_bias_E is None:
            raise ValueError(
                "Quantile-balanced routing requires an expert bias; the MoE "
                "owning this router must register expert_bias_E."
            )

    def _select_observing(self, logits_TE, expert_bias_E, padding_mask_T):
        """Biased top-(K+1) in one kernel, histogram accumulation in a second."""
        scores_TK, ids_TK, scores_TE, cutoff_T = Fn.route_select_cutoff(
            logits_TE, expert_bias_E, self.top_k, self.score_func, self.route_norm, float(self.route_scale)
        )
        self.quantile_balancer.observe(
            scores_TE.detach(), cutoff_T, expert_bias_E, padding_mask_T=padding_mask_T
        )
        return scores_TK, ids_TK, scores_TE, None

    def forward(self, x_TD, expert_bias_E=None, *, padding_mask_T=None):
        self._require_bias(expert_bias_E)
        return super().forward(x_TD, expert_bias_E, padding_mask_T=padding_mask_T)

    def route(self, x_TD, expert_bias_E=None, *, padding_mask_T=None):
        self._require_bias(expert_bias_E)
        if not self.training:
            return super().route(x_TD, expert_bias_E)
        if padding_mask_T is not None:
            padding_mask_T = padding_mask_T.reshape(-1)
        scores_TK, ids_TK, _, _ = self._select_observing(self.gate(x_TD), expert_bias_E, padding_mask_T)
        return scores_TK, ids_TK

    def _select(self, logits_TE, expert_bias_E, want_scores, padding_mask_T=None, want_map=False):
        self._require_bias(expert_bias_E)
        if not self.training:
            return super()._select(logits_TE, expert_bias_E, want_scores, want_map=want_map)
        return self._select_observing(logits_TE, expert_bias_E, padding_mask_T)
