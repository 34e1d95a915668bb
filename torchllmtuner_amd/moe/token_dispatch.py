"""Token dispatchers for one GPU: plan, row gather, weighted combine.

Interface of llmtuner/parallel/expert_parallel/token_dispatch.py:127-275
(``LocalTokenDispatcher``): ``dispatch(x_TD, topk_scores_TK, topk_expert_ids_TK,
num_local_tokens_per_expert_E) -> (routed_input_RD, counts_e, metadata)`` and
``combine(routed_output_RD, metadata, x_TD) -> out_TD``, plus ``num_experts``,
``top_k``, ``accumulate_in_fp32`` and ``set_ep_group``.

Two more dispatchers share the same kernels:

* ``PaddedTokenDispatcher`` -- the EP=1 behaviour of the reference's
  ``TorchAOTokenDispatcher`` (torchao_dispatch.py:82-185): each expert's rows are
  padded to a multiple of ``pad_multiple`` with zero rows, the padded counts are
  returned, and ``combine`` ignores the padding.  The layout is produced by the
  plan kernel itself; no third-party permute is involved.
* ``LocalShareTokenDispatcher`` -- one expert-parallel rank's share on one GPU:
  routing covers all experts, only experts ``[start, start + n)`` receive rows,
  the other assignments contribute nothing to the output but stay in the counts.

The rows are ordered exactly like ``argsort(ids.flatten(), stable=True)``.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from .. import functional as Fn
from .. import ops

__all__ = [
    "LocalDispatchMetadata",
    "LocalTokenDispatcher",
    "PaddedTokenDispatcher",
    "LocalShareTokenDispatcher",
]


@dataclass(frozen=True, kw_only=True)
class LocalDispatchMetadata:
    """What ``dispatch()`` hands to ``combine()``: the plan and the (T, K) scores."""

    plan: ops.PermutePlan
    topk_scores_TK: torch.Tensor

    @property
    def token_indices_experts_sorted_N(self) -> torch.Tensor:  # noqa: N802
        """Token of each row, int64 (-1 for padding rows); the reference's field."""
        slot = self.plan.slot_of_row.to(torch.int64)
        return torch.where(slot >= 0, slot // self.plan.top_k, slot)

    @property
    def topk_scores_experts_sorted_N(self) -> torch.Tensor:  # noqa: N802
        """Score of each row (0 for padding rows); the reference's field."""
        slot = self.plan.slot_of_row.to(torch.int64)
        flat = self.topk_scores_TK.reshape(-1)
        return torch.where(slot >= 0, flat[slot.clamp_min(0)], flat.new_zeros(()))


class LocalTokenDispatcher:
    """EP=1 dispatcher: local reordering only.  Not an ``nn.Module``."""

    def __init__(self, num_experts: int, top_k: int) -> None:
        self.num_experts = num_experts
        self.top_k = top_k
        self.accumulate_in_fp32 = False

    def set_ep_group(self, *, ep_group=None) -> None:
        """No-op: there is no expert-parallel group on one GPU."""
        del ep_group

    # -- layout knobs subclasses override --------------------------------------
    def _align(self) -> int:
        return 1

    def _local_range(self) -> tuple[int, int]:
        return 0, self.num_experts

    def _check_routing(self, x_TD, topk_scores_TK, topk_expert_ids_TK) -> None:
        if x_TD.ndim != 2:
            raise ValueError("Token inputs must have shape (tokens, hidden_dim)")
        routing_shape = (x_TD.shape[0], self.top_k)
        if tuple(topk_scores_TK.shape) != routing_shape or tuple(topk_expert_ids_TK.shape) != routing_shape:
            raise ValueError(
                "Routing scores and expert IDs must both have shape "
                f"{routing_shape}, matching the token count and top_k"
            )

    def plan(self, topk_expert_ids_TK: torch.Tensor) -> ops.PermutePlan:
        lo, hi = self._local_range()
        return ops.permute_plan(topk_expert_ids_TK, self.num_experts, lo, hi, self._align())

    def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        self._check_routing(x_TD, topk_scores_TK, topk_expert_ids_TK)
        plan = self.plan(topk_expert_ids_TK)
        rows = Fn.permute_rows(x_TD, plan)
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        return rows, num_local_tokens_per_expert_E, metadata

    def combine(self, routed_output_RD, metadata: LocalDispatchMetadata, x_TD):
        out = Fn.combine(
            routed_output_RD, metadata.topk_scores_TK, metadata.plan, not self.accumulate_in_fp32
        )
        return out.to(x_TD.dtype)


class PaddedTokenDispatcher(LocalTokenDispatcher):
    """Per-expert segments padded to a multiple of ``pad_multiple`` rows."""

    def __init__(self, num_experts: int, top_k: int, *, pad_multiple: int) -> None:
        super().__init__(num_experts, top_k)
        if not isinstance(pad_multiple, int) or isinstance(pad_multiple, bool) or pad_multiple < 1:
            raise ValueError(f"pad_multiple must be a positive integer, got {pad_multiple!r}")
        self.pad_multiple = pad_multiple

    def _align(self) -> int:
        return self.pad_multiple

    def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        self._check_routing(x_TD, topk_scores_TK, topk_expert_ids_TK)
        plan = self.plan(topk_expert_ids_TK)
        rows = Fn.permute_rows(x_TD, plan)
        # Resolving the covered size reads one int from the device, as the reference's
        # adapter does (torchao_dispatch.py:167).
        covered = int(plan.total_rows.item())
        padded_counts = (plan.seg_offsets[1:] - plan.seg_offsets[:-1]).to(torch.int64)
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        return rows[:covered], padded_counts, metadata


class LocalShareTokenDispatcher(LocalTokenDispatcher):
    """Rows only for experts ``[local_start, local_start + num_local_experts)``."""

    def __init__(self, num_experts: int, top_k: int, *, local_start: int, num_local_experts: int) -> None:
        super().__init__(num_experts, top_k)
        if not (0 <= local_start and num_local_experts >= 1 and local_start + num_local_experts <= num_experts):
            raise ValueError(
                f"local expert range [{local_start}, {local_start + num_local_experts}) "
                f"must lie inside [0, {num_experts})"
            )
        self.local_start = local_start
        self.num_local_experts = num_local_experts

    def _local_range(self) -> tuple[int, int]:
        return self.local_start, self.local_start + self.num_local_experts

    def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        self._check_routing(x_TD, topk_scores_TK, topk_expert_ids_TK)
        plan = self.plan(topk_expert_ids_TK)
        rows = Fn.permute_rows(x_TD, plan)
        covered = int(plan.total_rows.item())
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        return rows[:covered], plan.seg_counts.to(torch.int64), metadata
