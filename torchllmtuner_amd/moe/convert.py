"""Building the native block from HuggingFace-style packed expert tensors, and the
HF <-> native expert key mapping.

``moe_from_packed_experts`` follows what the reference's ``convert_block`` does once its
bindings are resolved (``llmtuner/parallel/expert_parallel/block_conversion.py:160-300``):
``gate_up_proj (E, 2F, D)`` splits along its output axis into ``w1_EFD`` (first F rows) and
``w3_EFD`` (last F rows), ``down_proj (E, D, F)`` is ``w2_EDF``, the router weight is copied
in its own dtype (fp32 under bf16 experts), the HF ``e_score_correction_bias`` seeds
``expert_bias_E`` and switches the auxiliary-loss-free bias update on, and an existing
shared-expert module is reused as is.  The key functions restate the format rules of
``llmtuner/models/qwen/qwen3/state.py:14-103``.
"""

from __future__ import annotations

import re
from collections.abc import Mapping

import torch
import torch.nn as nn

from .auxiliary_loss import MicrobatchWiseLoadBalanceLoss
from .experts import GroupedExperts, RoutedExperts
from .layer import MoE
from .routing import QuantileBalancedTopKRouter, TokenChoiceTopKRouter
from .token_dispatch import LocalShareTokenDispatcher, LocalTokenDispatcher, PaddedTokenDispatcher

__all__ = [
    "HF_PROJECTIONS",
    "NATIVE_PROJECTIONS",
    "convert_block",
    "hf_expert_state_to_native",
    "moe_from_packed_experts",
    "native_ep_expert_key",
    "native_expert_state_to_hf",
]

NATIVE_PROJECTIONS = {"gate_proj": "w1_EFD", "up_proj": "w3_EFD", "down_proj": "w2_EDF"}
HF_PROJECTIONS = {role: name for name, role in NATIVE_PROJECTIONS.items()}

_HF_EXPERT = re.compile(r"(.+\.mlp\.experts\.)(\d+)\.(gate_proj|up_proj|down_proj)\.weight")
_NATIVE_EXPERT = re.compile(r"(.+\.mlp\.)routed_experts\.inner_experts\.(w[123]_[A-Z]+)")


def native_ep_expert_key(key: str) -> str:
    """``….mlp.experts.7.up_proj.weight`` -> ``….mlp.routed_experts.inner_experts.w3_EFD``;
    any other key passes through (state.py:33-40)."""
    match = _HF_EXPERT.fullmatch(key)
    if match is None:
        return key
    return key.rsplit("experts.", 1)[0] + "routed_experts.inner_experts." + NATIVE_PROJECTIONS[match.group(3)]


def hf_expert_state_to_native(state: Mapping[str, torch.Tensor]) -> dict[str, torch.Tensor]:
    """Stack per-expert HF projections into the native ``(E, ., .)`` parameters.

    Every expert index 0..E-1 of a projection must be present; other keys are copied.
    """
    out: dict[str, torch.Tensor] = {}
    groups: dict[str, dict[int, torch.Tensor]] = {}
    for key, value in state.items():
        match = _HF_EXPERT.fullmatch(key)
        if match is None:
            out[key] = value
            continue
        groups.setdefault(native_ep_expert_key(key), {})[int(match.group(2))] = value
    for target, parts in groups.items():
        if sorted(parts) != list(range(len(parts))):
            raise ValueError(f"HF expert stack for {target} is incomplete: indices {sorted(parts)}")
        out[target] = torch.stack([parts[i] for i in range(len(parts))])
    return out


def native_expert_state_to_hf(state: Mapping[str, torch.Tensor], *, num_experts: int) -> dict[str, torch.Tensor]:
    """The inverse: one HF key per expert and projection (state.py:84-103); a partial
    stack cannot describe a complete external file."""
    out: dict[str, torch.Tensor] = {}
    for key, value in state.items():
        match = _NATIVE_EXPERT.fullmatch(key)
        if match is None:
            out[key] = value
            continue
        prefix, role = match.groups()
        if role not in HF_PROJECTIONS:
            raise ValueError(f"Unknown Qwen3 expert projection: {key}")
        if value.dim() != 3 or value.shape[0] != num_experts:
            raise ValueError(f"Qwen3 HF export requires full expert stack: {key}")
        for index in range(num_experts):
            out[f"{prefix}experts.{index}.{HF_PROJECTIONS[role]}.weight"] = value[index]
    return out


def moe_from_packed_experts(
    router_weight_ED: torch.Tensor,
    gate_up_proj_E2FD: torch.Tensor,
    down_proj_EDF: torch.Tensor,
    *,
    top_k: int,
    score_func: str = "softmax",
    route_norm: bool = False,
    route_scale: float = 1.0,
    num_expert_groups: int | None = None,
    num_limited_groups: int | None = None,
    e_score_correction_bias: torch.Tensor | None = None,
    load_balance_coeff: float = 1e-3,
    router_aux_loss_coef: float | None = None,
    shared_experts: nn.Module | None = None,
    token_dispatcher: str = "local",
    torchao_pad_multiple: int = 16,
    fixed_router: bool = False,
    local_experts: tuple[int, int] | None = None,
    training: bool = True,
) -> MoE:
    """One native block holding copies of the given packed tensors (on their device)."""
    if gate_up_proj_E2FD.dim() != 3 or down_proj_EDF.dim() != 3 or router_weight_ED.dim() != 2:
        raise ValueError("expected router (E,D), gate_up_proj (E,2F,D) and down_proj (E,D,F)")
    num_experts, dim = router_weight_ED.shape
    E_w, two_f, dim_w = gate_up_proj_E2FD.shape
    if two_f % 2 or dim_w != dim or down_proj_EDF.shape != (E_w, dim, two_f // 2):
        raise ValueError(
            f"packed expert shapes do not agree: gate_up {tuple(gate_up_proj_E2FD.shape)}, "
            f"down {tuple(down_proj_EDF.shape)}, router {tuple(router_weight_ED.shape)}"
        )
    hidden = two_f // 2
    lo, hi = (0, num_experts) if local_experts is None else local_experts
    if not (0 <= lo < hi <= num_experts) or E_w not in (num_experts, hi - lo):
        raise ValueError(f"local expert range {(lo, hi)} does not fit {E_w} packed experts of {num_experts}")
    if token_dispatcher not in ("local", "torchao"):
        raise ValueError(f"token_dispatcher {token_dispatcher!r} needs more than one process; use 'local' or 'torchao'")
    # the packed tensors hold either every expert or exactly the local ones
    take = slice(lo, hi) if E_w == num_experts else slice(None)

    grouped = GroupedExperts(dim, hidden, hi - lo)
    router = TokenChoiceTopKRouter(
        num_experts, dim, top_k, score_func=score_func, route_norm=route_norm, route_scale=route_scale,
        num_expert_groups=num_expert_groups, num_limited_groups=num_limited_groups,
        aux_loss=MicrobatchWiseLoadBalanceLoss(coeff=router_aux_loss_coef) if router_aux_loss_coef else None,
        fixed_router=fixed_router,
    )
    if local_experts is not None and (hi - lo) != num_experts:
        dispatcher = LocalShareTokenDispatcher(num_experts, top_k, local_start=lo, num_local_experts=hi - lo)
    elif token_dispatcher == "torchao":
        dispatcher = PaddedTokenDispatcher(num_experts, top_k, pad_multiple=torchao_pad_multiple)
    else:
        dispatcher = LocalTokenDispatcher(num_experts, top_k)
    moe = MoE(
        num_experts, RoutedExperts(grouped, dispatcher), router,
        # off for models that carry no bias buffer: a frozen zero bias is dead checkpoint state
        load_balance_coeff=load_balance_coeff if e_score_correction_bias is not None else None,
    )
    device = router_weight_ED.device
    moe.to(dtype=gate_up_proj_E2FD.dtype, device=device)
    router.to(dtype=router_weight_ED.dtype, device=device)
    with torch.no_grad():
        router.gate.weight.copy_(router_weight_ED)
        grouped.w1_EFD.copy_(gate_up_proj_E2FD[take, :hidden])
        grouped.w3_EFD.copy_(gate_up_proj_E2FD[take, hidden:])
        grouped.w2_EDF.copy_(down_proj_EDF[take])
        if e_score_correction_bias is not None:
            moe.expert_bias_E.copy_(e_score_correction_bias.float())
    router.gate.weight.requires_grad_(router_weight_ED.requires_grad)
    for target, source in ((grouped.w1_EFD, gate_up_proj_E2FD), (grouped.w3_EFD, gate_up_proj_E2FD),
                           (grouped.w2_EDF, down_proj_EDF)):
        target.requires_grad_(source.requires_grad)
    moe.shared_experts = shared_experts
    moe.train(training)
    return moe


def _expert_views(packed_experts, block):
    """(gate_EFD, up_EFD, down_EDF, num_experts) from whatever describes the packed experts: the
    reference's ``PackedExpertBinding`` (``projections(block)``, or its ``gate_up`` / ``down`` /
    ``shape`` fields) or its ``PackedExpertViews`` tuple (bindings.py:101-170), by their fields."""
    if hasattr(packed_experts, "gate_EFD"):
        views = packed_experts
    elif callable(getattr(packed_experts, "projections", None)):
        views = packed_experts.projections(block)
    elif hasattr(packed_experts, "gate_up") and hasattr(packed_experts, "down"):
        gate_up, down = packed_experts.gate_up, packed_experts.down
        hidden = gate_up.shape[1] // 2
        return gate_up[:, :hidden], gate_up[:, hidden:], down, gate_up.shape[0]
    else:
        raise TypeError(
            "packed_experts must provide gate_EFD / up_EFD / down_EDF / num_experts, a projections(block) "
            "method, or gate_up / down parameters"
        )
    return views.gate_EFD, views.up_EFD, views.down_EDF, int(views.num_experts)


def convert_block(
    block: nn.Module | None,
    *,
    routing,
    packed_experts,
    ep_group=None,
    aux_loss_coeff: float | None = None,
    load_balance_coeff: float | None = 1e-3,
    quantile_balancing: bool = False,
    token_dispatcher: str = "alltoall",
    torchao_pad_multiple: int = 16,
    tp_enabled: bool = False,
) -> MoE:
    """The reference's ``convert_block`` for one GPU, with its own keyword surface
    (llmtuner/parallel/expert_parallel/block_conversion.py:123-300): one native block built
    from already resolved bindings.

    ``routing`` is read by its fields (``router`` -- the HF gate module with ``weight (E, D)``
    and optionally ``e_score_correction_bias`` --, ``shared``, ``top_k``, ``score_func``,
    ``route_norm``, ``route_scale``, ``num_expert_groups``, ``num_limited_groups``; the reference's
    ``MoERoutingBinding``, bindings.py:36-98), ``packed_experts`` as described in
    ``_expert_views``; both are validated against ``block`` when they offer ``validate``.  No
    reference class is imported: any object with those fields will do.  One process owns every
    expert: an expert-parallel group, tensor parallelism and the dispatchers that need peers are
    refused.  ``block`` only supplies the training / eval mode (``None``: training).
    """
    if ep_group is not None:
        raise NotImplementedError("convert_block: this build runs on one GPU; ep_group must be None")
    if tp_enabled:
        raise NotImplementedError("convert_block: tensor parallelism needs more than one GPU")
    if token_dispatcher not in ("alltoall", "torchao"):
        raise NotImplementedError(
            f"convert_block: the {token_dispatcher!r} dispatcher needs expert-parallel peers; one GPU runs "
            "'alltoall' (local reordering at EP=1) or 'torchao' (padded segments)"
        )
    for binding in (routing, packed_experts):
        validate = getattr(binding, "validate", None)
        if callable(validate) and block is not None:
            validate(block)
    gate_EFD, up_EFD, down_EDF, num_experts = _expert_views(packed_experts, block)
    router_gate = routing.router
    weight = router_gate.weight
    if tuple(weight.shape) != (num_experts, gate_EFD.shape[2]):
        raise ValueError(
            f"router weight {tuple(weight.shape)} does not match {num_experts} experts of width {gate_EFD.shape[2]}"
        )
    dim, hidden, top_k = weight.shape[1], gate_EFD.shape[1], routing.top_k
    aux = MicrobatchWiseLoadBalanceLoss(coeff=aux_loss_coeff) if aux_loss_coeff else None
    if quantile_balancing:
        if routing.score_func != "sigmoid" or routing.num_expert_groups is not None:
            raise ValueError("quantile balancing is defined over sigmoid scores without expert groups")
        router = QuantileBalancedTopKRouter(num_experts, dim, top_k, route_norm=routing.route_norm,
                                            route_scale=routing.route_scale, aux_loss=aux)
        load_balance_coeff = None  # the quantile update owns expert_bias_E
    else:
        router = TokenChoiceTopKRouter(
            num_experts, dim, top_k, score_func=routing.score_func, route_norm=routing.route_norm,
            route_scale=routing.route_scale, num_expert_groups=routing.num_expert_groups,
            num_limited_groups=routing.num_limited_groups, aux_loss=aux)
    if token_dispatcher == "torchao":
        dispatcher = PaddedTokenDispatcher(num_experts, top_k, pad_multiple=torchao_pad_multiple)
    else:
        dispatcher = LocalTokenDispatcher(num_experts, top_k)
    grouped = GroupedExperts(dim, hidden, num_experts)
    moe = MoE(num_experts, RoutedExperts(grouped, dispatcher), router, load_balance_coeff=load_balance_coeff)
    # the expert subtree in its source dtype, the router in its own (fp32 under bf16 experts)
    moe.to(dtype=gate_EFD.dtype, device=weight.device)
    router.to(dtype=weight.dtype, device=weight.device)
    moe.train(True if block is None else block.training)
    projections = ((grouped.w1_EFD, gate_EFD), (grouped.w3_EFD, up_EFD), (grouped.w2_EDF, down_EDF))
    router.gate.weight.requires_grad_(weight.requires_grad)
    for target, source in projections:
        target.requires_grad_(source.requires_grad)
    with torch.no_grad():
        router.gate.weight.copy_(weight)
        for target, source in projections:
            target.copy_(source)
        bias = getattr(router_gate, "e_score_correction_bias", None)
        if bias is not None and moe.expert_bias_E is not None:
            moe.expert_bias_E.copy_(bias.float())
    # the HF shared expert is reused as it is, after the new subtree was cast and moved
    moe.shared_experts = getattr(routing, "shared", None)
    return moe
