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

import weakref

import torch

from .. import ops as Fn
from .. import ops

__all__ = [
    "LocalDispatchMetadata",
    "LocalTokenDispatcher",
    "PaddedTokenDispatcher",
    "LocalShareTokenDispatcher",
]


class LocalDispatchMetadata:
    """What ``dispatch()`` hands to ``combine()``.

    The reference's record has two fields (token_dispatch.py:84-89):
    ``token_indices_experts_sorted_N`` (token of each expert-sorted row) and
    ``topk_scores_experts_sorted_N`` (score of each row); both are accepted as keywords and
    readable here.  Records made by this package's dispatchers also carry the permutation
    ``plan`` and the unsorted ``(T, K)`` scores, which is what the device kernels consume;
    the two reference fields are then derived from the plan on first access (-1 / 0 for
    padding rows).
    """

    __slots__ = ("plan", "topk_scores_TK", "_token_indices", "_scores_sorted")

    def __init__(self, *, token_indices_experts_sorted_N: torch.Tensor | None = None,
                 topk_scores_experts_sorted_N: torch.Tensor | None = None,
                 plan: ops.PermutePlan | None = None, topk_scores_TK: torch.Tensor | None = None) -> None:
        if plan is None and (token_indices_experts_sorted_N is None or topk_scores_experts_sorted_N is None):
            raise TypeError(
                "LocalDispatchMetadata needs token_indices_experts_sorted_N and "
                "topk_scores_experts_sorted_N (or a plan with the (T, K) scores)"
            )
        if plan is not None and topk_scores_TK is None:
            raise TypeError("LocalDispatchMetadata: a plan needs the (T, K) scores it was made for")
        self.plan = plan
        self.topk_scores_TK = topk_scores_TK
        self._token_indices = token_indices_experts_sorted_N
        self._scores_sorted = topk_scores_experts_sorted_N

    @property
    def token_indices_experts_sorted_N(self) -> torch.Tensor:  # noqa: N802
        """Token of each row, int64 (-1 for padding rows)."""
        if self._token_indices is None:
            slot = self.plan.slot_of_row.to(torch.int64)
            self._token_indices = torch.where(slot >= 0, slot // self.plan.top_k, slot)
        return self._token_indices

    @property
    def topk_scores_experts_sorted_N(self) -> torch.Tensor:  # noqa: N802
        """Score of each row (0 for padding rows)."""
        if self._scores_sorted is None:
            slot = self.plan.slot_of_row.to(torch.int64)
            flat = self.topk_scores_TK.reshape(-1)
            self._scores_sorted = torch.where(slot >= 0, flat[slot.clamp_min(0)], flat.new_zeros(()))
        return self._scores_sorted


class LocalTokenDispatcher:
    """EP=1 dispatcher: local reordering only.  Not an ``nn.Module``."""

    def __init__(self, num_experts: int, top_k: int) -> None:
        self.num_experts = num_experts
        self.top_k = top_k
        self.accumulate_in_fp32 = False
        # combine() of a record that carries only the reference's two fields checks that every
        # token owns exactly top_k rows; the check reads one flag back from the device (a host
        # synchronisation) and can be switched off by callers who build such records themselves
        self.validate_foreign_records = True
        self._last_plan = None  # (weakref to the ids tensor, its version, the plan made for it, its layout key)

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
        """The expert-major layout for these ids.  The plan of the most recent call is kept
        and returned again for the very same tensor object (unchanged since): the block asks
        for the counts first and the experts for the layout right after."""
        ids = topk_expert_ids_TK
        lo, hi = self._local_range()
        layout = (self.num_experts, lo, hi, self._align())
        if torch.compiler.is_compiling():
            # no memo under a tracing compiler: it would keep traced tensors in module state, and a
            # tensor's version counter is not a value the trace can branch on
            return ops.permute_plan(ids, self.num_experts, lo, hi, self._align())
        last = self._last_plan
        if last is not None and last[0]() is ids and last[1] == ids._version and last[3] == layout:
            return last[2]
        plan = ops.permute_plan(ids, self.num_experts, lo, hi, self._align())
        try:
            self._last_plan = (weakref.ref(ids), ids._version, plan, layout)
        except TypeError:  # tensor subclasses without weak references: no memo
            self._last_plan = None
        return plan

    def forget_plan(self) -> None:
        """Drop the kept plan (its index arrays are N-sized); the next ``plan()`` builds anew."""
        self._last_plan = None

    def _permute_tokens(self, inputs, token_indices, expert_ids):
        """Gather tokens into expert-major rows -- the hook of token_dispatch.py:197-199
        ("backend adapters may own the repeated-index VJP").  This class's own gather is the
        plan's row kernel, whose backward is the K-way row sum in a fixed order; it takes the
        layout from the plan of ``expert_ids`` and does not read ``token_indices`` (``dispatch``
        passes None here and the token of every row, int64 with -1 for padding rows, to an
        override)."""
        del token_indices
        return Fn.permute_rows(inputs, self.plan(expert_ids))

    def _gather_rows(self, x_TD, topk_expert_ids_TK, metadata: "LocalDispatchMetadata"):
        overridden = type(self)._permute_tokens is not LocalTokenDispatcher._permute_tokens
        token_indices = metadata.token_indices_experts_sorted_N if overridden else None
        return self._permute_tokens(x_TD, token_indices, topk_expert_ids_TK)

    def _rows_for_combine(self, routed_output_RD, metadata: "LocalDispatchMetadata"):
        """(plan, scores_TK) for a record that only carries the reference's two fields: with
        K rows per token the stable order of the token indices IS the slot -> row map."""
        tok = metadata.token_indices_experts_sorted_N
        K = self.top_k
        if tok.numel() % K != 0:
            raise ValueError("combine: the dispatch record does not hold top_k rows per token")
        T = tok.numel() // K
        order = torch.argsort(tok, stable=True)
        if self.validate_foreign_records and T > 0 and not bool(
                (tok[order].view(T, K) == torch.arange(T, device=tok.device)[:, None]).all()):
            raise ValueError("combine: the dispatch record does not hold top_k rows per token")
        row_of_slot = order.to(torch.int32)
        inv = torch.empty_like(row_of_slot)
        inv[order] = torch.arange(tok.numel(), device=tok.device, dtype=torch.int32)
        counts = torch.tensor([tok.numel()], dtype=torch.int32, device=tok.device)
        seg = ops.segments_from_counts(counts, tok.numel())
        plan = ops.PermutePlan(T, K, 1, 0, 1, 1, seg.tile_m, tok.numel(), seg.tile_capacity, None, seg.seg_offsets,
                               seg.seg_counts, row_of_slot, inv, None, seg.tile_expert, seg.tile_row0,
                               seg.num_tiles, seg.expert_order)
        return plan, metadata.topk_scores_experts_sorted_N[order].view(T, K)

    def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        self._check_routing(x_TD, topk_scores_TK, topk_expert_ids_TK)
        plan = self.plan(topk_expert_ids_TK)
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        rows = self._gather_rows(x_TD, topk_expert_ids_TK, metadata)
        return rows, num_local_tokens_per_expert_E, metadata

    def combine(self, routed_output_RD, metadata: LocalDispatchMetadata, x_TD):
        if metadata.plan is not None:
            plan, scores_TK = metadata.plan, metadata.topk_scores_TK
        else:
            plan, scores_TK = self._rows_for_combine(routed_output_RD, metadata)
        out = Fn.combine(routed_output_RD, scores_TK, plan, not self.accumulate_in_fp32)
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
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        rows = self._gather_rows(x_TD, topk_expert_ids_TK, metadata)
        # Resolving the covered size reads one int from the device, as the reference's
        # adapter does (torchao_dispatch.py:167).
        covered = int(plan.total_rows.item())
        padded_counts = (plan.seg_offsets[1:] - plan.seg_offsets[:-1]).to(torch.int64)
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
        metadata = LocalDispatchMetadata(plan=plan, topk_scores_TK=topk_scores_TK)
        rows = self._gather_rows(x_TD, topk_expert_ids_TK, metadata)
        covered = int(plan.total_rows.item())
        return rows[:covered], plan.seg_counts.to(torch.int64), metadata
