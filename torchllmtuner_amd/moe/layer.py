"""The MoE block: route, dispatch, expert compute, combine, (shared experts), sum.

Drop-in for llmtuner/models/common/moe/layer.py:88-309 (``MoE``): same
constructor, same module tree and state-dict keys (``router.gate.weight``,
``routed_experts.inner_experts.{w1_EFD,w3_EFD,w2_EDF}``, persistent fp32 buffer
``expert_bias_E``, non-persistent fp32 buffer ``tokens_per_expert_E``,
``shared_experts.*``), same ``forward(x, *, padding_mask=None)`` contract
including ``(..., T, D)`` inputs, staged padding masks, training-only counters
committed after both expert paths succeed, and ``returns_router_logits``.
"""

from __future__ import annotations

import math
from collections.abc import Iterator
from numbers import Real

import torch
import torch.nn as nn

from .. import ops
from .auxiliary_loss import in_checkpoint_recompute
from .experts import RoutedExperts, _is_own_dispatcher
from .routing import QuantileBalancedTopKRouter, TokenChoiceTopKRouter

__all__ = ["MoE", "in_checkpoint_recompute"]

# in_checkpoint_recompute is set by an activation-checkpointing wrapper while it replays a
# forward; counter updates are skipped there (llmtuner/models/common/aux_loss.py:47-68).


class MoE(nn.Module):
    def __init__(
        self,
        num_experts: int,
        routed_experts: RoutedExperts,
        router: TokenChoiceTopKRouter,
        *,
        load_balance_coeff: float | None = 1e-3,
        shared_experts: nn.Module | None = None,
    ) -> None:
        super().__init__()
        if not isinstance(num_experts, int) or isinstance(num_experts, bool) or num_experts < 1:
            raise ValueError("num_experts must be a positive integer")
        if num_experts != router.num_experts:
            raise ValueError(
                f"MoE num_experts ({num_experts}) must match router.num_experts ({router.num_experts})"
            )
        dispatcher = routed_experts.token_dispatcher
        if dispatcher is None:
            raise ValueError("MoE routed experts require a token dispatcher")
        if dispatcher.num_experts != num_experts:
            raise ValueError(
                "MoE dispatcher.num_experts must match router.num_experts; "
                f"got {dispatcher.num_experts} and {num_experts}"
            )
        if dispatcher.top_k != router.top_k:
            raise ValueError(
                f"MoE dispatcher.top_k must match router.top_k; got {dispatcher.top_k} and {router.top_k}"
            )
        quantile_balanced = isinstance(router, QuantileBalancedTopKRouter)
        if quantile_balanced and load_balance_coeff is not None:
            raise ValueError(
                "A QuantileBalancedTopKRouter is balanced by the quantile "
                "update, so load_balance_coeff must be None -- the sign-based "
                "and quantile updates cannot both own expert_bias_E."
            )
        if load_balance_coeff is not None and (
            not isinstance(load_balance_coeff, Real)
            or isinstance(load_balance_coeff, bool)
            or not math.isfinite(load_balance_coeff)
            or load_balance_coeff <= 0.0
        ):
            raise ValueError(f"load_balance_coeff must be finite and positive, got {load_balance_coeff}")
        self.routed_experts = routed_experts
        self.router = router
        self.shared_experts = shared_experts
        self.load_balance_coeff = load_balance_coeff
        # both balancing schemes persist the balance they reached (layer.py:169-177)
        if load_balance_coeff is not None or quantile_balanced:
            self.register_buffer(
                "expert_bias_E", torch.zeros(num_experts, dtype=torch.float32), persistent=True
            )
        else:
            self.expert_bias_E = None
        self.register_buffer(
            "tokens_per_expert_E", torch.zeros(num_experts, dtype=torch.float32), persistent=False
        )
        self._pending_padding_mask: torch.Tensor | None = None
        self.returns_router_logits = False
        # The shared expert reads nothing but the tokens: it runs on a second stream beside the
        # router, the plan and the routed experts (their small kernels and memory-bound tiles
        # leave most of the matrix cores idle), and autograd runs its backward there as well.
        # Set to False to keep everything on the caller's stream.
        self.overlap_shared_experts = True

    # The two statistics buffers stay fp32 when the block is cast to bf16
    # (llmtuner/parallel/expert_parallel/block_conversion.py:61-79).
    def _apply(self, fn, *args, **kwargs):
        keep = {
            name: getattr(self, name)
            for name in ("expert_bias_E", "tokens_per_expert_E")
            if isinstance(getattr(self, name, None), torch.Tensor)
        }
        super()._apply(fn, *args, **kwargs)
        for name, old in keep.items():
            new = getattr(self, name)
            if new.dtype != torch.float32:
                self._buffers[name] = old.to(device=new.device, dtype=torch.float32)
        return self

    def expert_parallel_parameters(self) -> Iterator[nn.Parameter]:
        yield from self.routed_experts.inner_experts.parameters()

    @torch.no_grad()
    def update_expert_bias(self) -> None:
        """Sign-based, mean-centred bias nudge from the accumulated counts (layer.py:204-228)."""
        if self.expert_bias_E is None or self.load_balance_coeff is None:
            return
        counts_E = self.tokens_per_expert_E
        delta_E = self.load_balance_coeff * torch.sign(counts_E.mean() - counts_E)
        self.expert_bias_E.add_(delta_E - delta_E.mean())
        self.tokens_per_expert_E.zero_()

    def _start_shared_experts(self, tokens: torch.Tensor):
        """Launch the shared expert on the library's second stream, behind everything the
        caller's stream holds so far.  Returns ``(output, stream)``, or ``(None, None)`` when the
        shared expert is to run in place (none, switched off, not a real device tensor, under a
        tracing compiler, or no second stream yet -- its first use must not be under capture)."""
        if (
            self.shared_experts is None
            or not self.overlap_shared_experts
            or not tokens.is_cuda
            or isinstance(tokens, torch._subclasses.FakeTensor)
            or torch.compiler.is_compiling()
        ):
            return None, None
        stream = ops.aux_stream(tokens.device)
        if stream is None:
            return None, None
        stream.wait_stream(torch.cuda.current_stream(tokens.device))
        if tokens.is_leaf and tokens.requires_grad:
            # a leaf's gradient accumulator belongs to the stream of the leaf's first use: make
            # that the caller's stream (a view, no kernel), not the second one
            tokens = tokens.view_as(tokens)
        with torch.cuda.stream(stream):
            shared_TD = self.shared_experts(tokens)
        return shared_TD, stream

    def set_padding_mask(self, padding_mask: torch.Tensor | None) -> None:
        self._pending_padding_mask = padding_mask

    def forward(self, x: torch.Tensor, *, padding_mask: torch.Tensor | None = None):
        if padding_mask is None:
            padding_mask = self._pending_padding_mask
        restore_shape = x.dim() > 2
        tokens = x.reshape(-1, x.shape[-1]) if restore_shape else x
        if restore_shape and padding_mask is not None:
            padding_mask = padding_mask.reshape(-1)
        if padding_mask is not None:
            if padding_mask.dtype != torch.bool:
                raise ValueError(f"padding_mask_T must have dtype bool, got {padding_mask.dtype}.")
            if padding_mask.shape != tokens.shape[:-1]:
                raise ValueError(
                    "padding_mask_T must have shape matching the routing-map token axis, "
                    f"got {tuple(padding_mask.shape)} for {tokens.shape[0]} tokens."
                )

        shared_TD, shared_stream = self._start_shared_experts(tokens)

        topk_scores_TK, topk_expert_ids_TK, routing_map_TE = self.router(
            tokens, self.expert_bias_E, padding_mask_T=padding_mask
        )
        # The reference counts by summing the routing map (layer.py:278); the permutation plan
        # counts the same slots on the device as a by-product, and the dispatcher hands that
        # very plan to the experts a moment later, so neither the sum nor a second plan is run.
        # A dispatcher that is not this package's own (anything that only implements the
        # dispatch / combine protocol, token_dispatch.py:201-275) has no plan: the counts are then
        # the column sums of the routing map, as in the reference.
        dispatcher = self.routed_experts.token_dispatcher
        if _is_own_dispatcher(dispatcher):
            num_tokens_per_expert_E = dispatcher.plan(topk_expert_ids_TK).counts_E
        else:
            num_tokens_per_expert_E = routing_map_TE.sum(dim=0)
        out_TD = self.routed_experts(tokens, topk_scores_TK, topk_expert_ids_TK, num_tokens_per_expert_E)

        if shared_stream is not None:
            # join: the caller's stream waits for the shared expert, whose output (allocated on
            # the other stream) is marked as used here so that its memory is not handed out early
            main = torch.cuda.current_stream(tokens.device)
            main.wait_stream(shared_stream)
            shared_TD.record_stream(main)
            out_TD = out_TD + shared_TD
        elif self.shared_experts is not None:
            out_TD = out_TD + self.shared_experts(tokens)
        # Commit this block's observations only after both expert paths succeeded.
        # (a tracing compiler runs this once and replays the graph, recomputation included, without
        # re-entering the module: there is no recompute pass to skip, and it cannot read the context
        # variable)
        if self.training and (torch.compiler.is_compiling() or not in_checkpoint_recompute.get()):
            with torch.no_grad():
                if padding_mask is None:
                    valid_counts_E = num_tokens_per_expert_E  # int32; add_ promotes inside its one kernel
                else:
                    keep = (~padding_mask).to(torch.float32).repeat_interleave(topk_expert_ids_TK.shape[-1])
                    valid_counts_E = torch.zeros_like(self.tokens_per_expert_E).scatter_add_(
                        0, topk_expert_ids_TK.reshape(-1), keep
                    )
                self.tokens_per_expert_E.add_(valid_counts_E)

        if restore_shape:
            out_TD = out_TD.reshape(*x.shape[:-1], out_TD.shape[-1])
        return (out_TD, None) if self.returns_router_logits else out_TD
