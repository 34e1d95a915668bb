"""Expert weights and the routed-expert module, on the grouped expert kernels.

Constructor surface, parameter names and validation of
llmtuner/models/common/moe/experts.py:73-343 (``GroupedExperts``,
``RoutedExperts``, ``DispatchObservation``, ``ExpertErrorCapture``).  The three
stacked parameters keep their names and layouts -- ``w1_EFD`` and ``w3_EFD`` of
shape ``(E, F, D)``, ``w2_EDF`` of shape ``(E, D, F)`` -- so a reference state
dict loads key for key.

``RoutedExperts.forward`` keeps the reference signature and chooses the device path
itself: where the fused kernels apply (bf16, MFMA-sized widths) the row gather rides in
the expert GEMMs' operand loads and the combine's backward in their backward; otherwise
dispatch, experts and combine run as separate stages.  Nothing here synchronises the
host with the device.
"""

from __future__ import annotations

from contextlib import AbstractContextManager, nullcontext
from dataclasses import dataclass
import types
from typing import Protocol

import torch
import torch.nn as nn

from .. import ops as Fn
from .. import ops
from .activation import SwiGLU

__all__ = [
    "DenseSwiGLU",
    "DispatchObservation",
    "ExpertErrorCapture",
    "GroupedExperts",
    "RoutedExperts",
]


class DispatchObserver(Protocol):
    def measure(self, device: torch.device) -> AbstractContextManager[None]: ...


@dataclass(eq=False, slots=True)
class DispatchObservation:
    """Optional observation boundary entered by the expert dispatch forward."""

    observer: DispatchObserver | None = None

    def measure(self, device: torch.device) -> AbstractContextManager[None]:
        return nullcontext() if self.observer is None else self.observer.measure(device)


@dataclass
class ExpertErrorCapture:
    """Carries a local compute error past module hooks; check ``error`` before use."""

    error: BaseException | None = None


class GroupedExperts(nn.Module):
    """All experts' weights as three ``(E, O, I)`` tensors."""

    def __init__(
        self,
        dim: int,
        hidden_dim: int,
        num_experts: int,
        *,
        activation_fn: nn.Module | None = None,
        use_grouped_mm: bool | None = None,
    ) -> None:
        super().__init__()
        for name, value in (("dim", dim), ("hidden_dim", hidden_dim), ("num_experts", num_experts)):
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ValueError(f"{name} must be positive integer, got {value!r}")
        if use_grouped_mm is not None and not isinstance(use_grouped_mm, bool):
            raise TypeError("use_grouped_mm must be bool or None")
        self.num_experts = num_experts
        self.hidden_dim = hidden_dim
        self.dim = dim
        # Kept for interface parity; the device path always runs the grouped kernels.
        self.use_grouped_mm = True if use_grouped_mm is None else use_grouped_mm
        self.activation_fn = activation_fn if activation_fn is not None else SwiGLU()
        self._call_plan = None  # (plan, zero_fill) while compute_planned runs its grouped products
        self.w1_EFD = nn.Parameter(torch.empty(num_experts, hidden_dim, dim))
        self.w3_EFD = nn.Parameter(torch.empty(num_experts, hidden_dim, dim))
        self.w2_EDF = nn.Parameter(torch.empty(num_experts, dim, hidden_dim))

    def forward(self, x_RD, num_tokens_per_expert_E, *, error_capture: ExpertErrorCapture | None = None):
        if error_capture is None:
            return self._compute(x_RD, num_tokens_per_expert_E)
        error_capture.error = None
        try:
            return self._compute(x_RD, num_tokens_per_expert_E)
        except BaseException as error:  # noqa: BLE001 - deferred to the caller by contract
            error_capture.error = error
            return x_RD.detach()

    def _weights_as(self, dtype):
        cast = lambda w: w if w.dtype == dtype else w.to(dtype)
        return cast(self.w1_EFD), cast(self.w3_EFD), cast(self.w2_EDF)

    def _compute(self, x_RD, num_tokens_per_expert_E):
        if x_RD.ndim != 2 or x_RD.shape[1] != self.dim:
            raise ValueError(
                f"Expert inputs must have shape (routed_tokens, {self.dim}), got {tuple(x_RD.shape)}"
            )
        if x_RD.shape[0] > torch.iinfo(torch.int32).max:
            raise ValueError("Routed token count exceeds int32 grouped GEMM offsets")
        if tuple(num_tokens_per_expert_E.shape) != (self.num_experts,):
            raise ValueError(
                f"Expert token counts must have shape ({self.num_experts},), "
                f"got {tuple(num_tokens_per_expert_E.shape)}"
            )
        if num_tokens_per_expert_E.dtype not in (
            torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
        ):
            raise TypeError("Expert token counts must use an integer dtype")
        # Counts are clamped on the device (negatives to zero, segments to the rows that
        # exist), so malformed counts cannot make a kernel read out of bounds; rows that the
        # counts do not cover come back as zeros (and get zero gradients).
        plan = ops.segments_from_counts(num_tokens_per_expert_E, x_RD.shape[0])
        return self.compute_planned(x_RD, plan, zero_fill=True)

    def _grouped_mm(self, x_TD, weight_EOI, offsets_E):
        """``x . weight[e]^T`` per expert segment: the reference's pluggable product, with its
        signature (experts.py:211-216).  ``offsets_E`` are the segments' end offsets (int32), the
        cumulative counts the reference passes to ``torch._grouped_mm``; this implementation
        reads the same segments from the plan of the call in progress, which also carries the
        tile list the kernels walk.  An override receives exactly the reference's arguments."""
        plan, zero_fill = self._call_plan
        return Fn.grouped_linear(x_TD, weight_EOI, plan, zero_fill=zero_fill)

    def fuses_activation(self) -> bool:
        """SwiGLU exactly (not a subclass that may compute something else) is evaluated inside
        the gate/up kernel; any other gated activation, and any subclass that brings its own
        ``_grouped_mm``, runs as three grouped linear maps with the activation between them."""
        if type(self)._grouped_mm is not GroupedExperts._grouped_mm:
            return False  # a subclass's own grouped product must be the one that runs
        cls = type(self.activation_fn)
        # (the reference's own class, llmtuner.models.common.activation.SwiGLU, is the same function)
        return cls is SwiGLU or (cls.__name__ == "SwiGLU" and cls.__module__.endswith("models.common.activation"))

    def compute_planned(self, x_RD, plan: ops.PermutePlan, zero_fill: bool = False):
        w1, w3, w2 = self._weights_as(x_RD.dtype)
        if self.fuses_activation():
            return Fn.grouped_swiglu(x_RD, w1, w3, w2, plan, zero_fill=zero_fill)
        # experts.py:204-209 with the caller's activation: gate, up, activation(gate, up), down
        offsets_E = plan.seg_offsets[1:]
        self._call_plan = (plan, zero_fill)  # (one call at a time per module, like any forward)
        try:
            gate = self._grouped_mm(x_RD, w1, offsets_E)
            up = self._grouped_mm(x_RD, w3, offsets_E)
            h = self.activation_fn(gate, up)
            return self._grouped_mm(h, w2, offsets_E).type_as(x_RD)
        finally:
            self._call_plan = None


class RoutedExperts(nn.Module):
    """The dispatch/combine pair wrapped around the grouped expert weights."""

    def __init__(self, grouped_experts: GroupedExperts, dispatcher) -> None:
        super().__init__()
        self.inner_experts = grouped_experts
        self.token_dispatcher = dispatcher
        self.dispatch_observation = DispatchObservation() if type(self) is RoutedExperts else None

    def forward(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        """Dispatch tokens to experts, run them, and combine the results."""
        dispatcher = self.token_dispatcher
        experts = self.inner_experts
        observe = (
            self.dispatch_observation.measure(x_TD.device)
            if self.dispatch_observation is not None
            else nullcontext()
        )
        if not _is_own_dispatcher(dispatcher):
            # Any other dispatcher is driven through the protocol alone, exactly as
            # llmtuner/models/common/moe/experts.py:321-343 does: dispatch -> experts -> combine.
            # That covers objects that implement only dispatch / combine and subclasses of this
            # package's dispatchers that override dispatch, combine, plan or _permute_tokens.
            with observe:
                rows, counts_e, metadata = dispatcher.dispatch(
                    x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E
                )
            return dispatcher.combine(experts(rows, counts_e), metadata, x_TD)
        # This package's own dispatchers: the counts handed in are the plan's own (MoE.forward
        # takes them from the same plan), so the layout is read from the plan directly.
        dispatcher._check_routing(x_TD, topk_scores_TK, topk_expert_ids_TK)
        round_terms = not dispatcher.accumulate_in_fp32
        fused = (
            _is_plain_grouped_experts(experts)  # hooks on, or a subclass of, the inner module must run
            and experts.fuses_activation()
            and ops.gather_supported(x_TD, experts.hidden_dim)
            and x_TD.is_contiguous()
            and ops.combine_bwd_slots(x_TD.dtype, x_TD.shape[-1], experts.hidden_dim) > 0
        )
        try:
            if fused:
                # the dispatch is the plan alone: the row gather rides inside the expert kernels'
                # operand loads, and the combine's backward inside their backward
                with observe:
                    plan = dispatcher.plan(topk_expert_ids_TK)
                w1, w3, w2 = experts._weights_as(x_TD.dtype)
                out = Fn.gather_experts_combine(x_TD, topk_scores_TK, w1, w3, w2, plan, round_terms)
                return out.to(x_TD.dtype)
            if _is_plain_grouped_experts(experts) and experts.fuses_activation():
                # the same three stages as below as one operator each way: one trip through the
                # dispatcher and one autograd node, which is most of a small step's time
                with observe:
                    plan = dispatcher.plan(topk_expert_ids_TK)
                w1, w3, w2 = experts._weights_as(x_TD.dtype)
                out = Fn.rows_experts_combine(x_TD, topk_scores_TK, w1, w3, w2, plan, round_terms)
                return out.to(x_TD.dtype)
            with observe:
                plan = dispatcher.plan(topk_expert_ids_TK)
                rows = Fn.permute_rows(x_TD, plan)
            if _is_plain_grouped_experts(experts):
                # nothing hangs on the inner module's call: the experts run on the dispatcher's own
                # plan (no second plan from counts, no count arithmetic; padding rows belong to no
                # segment, are not computed and are never read by the combine)
                y = experts.compute_planned(rows, plan)
            else:
                # rows per local expert as laid out (padding included), the counts the reference hands
                # to its inner module; rows past the last segment are not covered and come back as zeros
                covered = plan.seg_offsets[1:] - plan.seg_offsets[:-1]
                y = experts(rows, covered)
            out = Fn.combine(y, topk_scores_TK, plan, round_terms)
            return out.to(x_TD.dtype)
        finally:
            # the plan lives on in the autograd graph as long as a backward needs it; the
            # dispatcher's own reference would keep its N-sized index arrays until the next step
            dispatcher.forget_plan()


def _is_own_dispatcher(dispatcher) -> bool:
    """True when ``dispatcher`` is one of this package's dispatchers with ``dispatch``, ``combine``,
    ``plan`` and ``_permute_tokens`` as this package defines them (a subclass that overrides none
    of them included): only then may RoutedExperts.forward replace the three protocol calls by
    the planned / fused kernels, which compute the same thing."""
    cls = type(dispatcher)
    seams = (getattr(cls, "dispatch", None), getattr(cls, "combine", None), getattr(cls, "plan", None),
             getattr(cls, "_permute_tokens", None))
    own = _OWN_DISPATCHER_CLASSES.get(seams)  # keyed by the functions themselves: a class patched later misses
    if own is None:
        from . import token_dispatch as td

        base = td.LocalTokenDispatcher
        own_dispatch = {c.__dict__["dispatch"] for c in (base, td.PaddedTokenDispatcher, td.LocalShareTokenDispatcher)}
        own = (
            issubclass(cls, base)
            and getattr(cls, "dispatch", None) in own_dispatch
            and cls.combine is base.combine
            and cls.plan is base.plan
            and cls._permute_tokens is base._permute_tokens
        )
        _OWN_DISPATCHER_CLASSES[seams] = own
    if not own:
        return False
    # methods patched onto the instance count as overrides too: what the instance hands out must be the
    # class's function bound to it (written so that a tracing compiler can follow it: no instance dictionary)
    dispatch, combine, plan, permute = (dispatcher.dispatch, dispatcher.combine, dispatcher.plan,
                                        dispatcher._permute_tokens)
    return (
        isinstance(dispatch, types.MethodType) and dispatch.__func__ is cls.dispatch
        and isinstance(combine, types.MethodType) and combine.__func__ is cls.combine
        and isinstance(plan, types.MethodType) and plan.__func__ is cls.plan
        and isinstance(permute, types.MethodType) and permute.__func__ is cls._permute_tokens
    )


_OWN_DISPATCHER_CLASSES: dict = {}  # a class's four seam methods -> whether they are this package's own


def _is_plain_grouped_experts(module: nn.Module) -> bool:
    """True when calling the module is exactly GroupedExperts._compute: no subclass override
    and no hook anywhere that a caller could be relying on."""
    from torch.nn.modules import module as _m

    cls = type(module)
    if cls.forward is not GroupedExperts.forward or cls._compute is not GroupedExperts._compute:
        return False
    own = (module._forward_hooks, module._forward_pre_hooks, module._backward_hooks, module._backward_pre_hooks)
    shared = (_m._global_forward_hooks, _m._global_forward_pre_hooks, _m._global_backward_hooks,
              _m._global_backward_pre_hooks)
    return not any(own) and not any(shared)


class DenseSwiGLU(nn.Module):
    """A dense SwiGLU MLP (the shared expert) on the same grouped kernels, E = 1.

    Parameter names follow the HF MLP the reference reuses as the shared expert
    (llmtuner/parallel/expert_parallel/block_conversion.py:278-291):
    ``gate_proj.weight (F, D)``, ``up_proj.weight (F, D)``, ``down_proj.weight (D, F)``.
    """

    def __init__(self, dim: int, hidden_dim: int) -> None:
        super().__init__()
        self.gate_proj = nn.Linear(dim, hidden_dim, bias=False)
        self.up_proj = nn.Linear(dim, hidden_dim, bias=False)
        self.down_proj = nn.Linear(hidden_dim, dim, bias=False)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, x.shape[-1])
        counts = torch.full((1,), x2.shape[0], dtype=torch.int32, device=x2.device)
        plan = ops.segments_from_counts(counts, x2.shape[0])
        dt = x2.dtype
        cast = lambda w: (w if w.dtype == dt else w.to(dt)).unsqueeze(0)
        y = Fn.grouped_swiglu(
            x2, cast(self.gate_proj.weight), cast(self.up_proj.weight), cast(self.down_proj.weight), plan
        )
        return y.reshape(*lead, y.shape[-1])
