"""Per-optimizer-step expert-bias updates of the MoE blocks.

Single-process form of llmtuner/models/common/moe/bias_update.py:26-288: the sign-based
update (``MoE.update_expert_bias``) and the quantile-histogram update share one
policy-selection entry point, ``register_moe_balancing_hook``, which validates that every
block of the model uses the same scheme and registers one optimizer step pre-hook.  The
reference sums the counters and histograms over the data-, context- and (under expert
parallelism) tensor-parallel axes first; with one process there is nothing to sum, so
``parallel_dims`` must be ``None``.  Blocks are found by walking the modules (the
reference reads its whole-model ``DecoderStructure`` declaration, which is not part of
this package).
"""

from __future__ import annotations

from collections.abc import Sequence

import torch
import torch.nn as nn

from .layer import MoE
from .routing import QuantileBalancedTopKRouter

__all__ = [
    "collect_moe_layers",
    "collect_routing_load_metrics",
    "register_moe_balancing_hook",
    "reset_routing_statistics",
    "update_expert_bias",
    "update_quantile_expert_bias",
]


def _single_process(parallel_dims) -> None:
    if parallel_dims is not None:
        raise NotImplementedError(
            "statistics are not reduced across processes in this build; pass parallel_dims=None"
        )


def collect_moe_layers(model_parts: Sequence[nn.Module]) -> list[MoE]:
    """Distinct MoE blocks of the model parts, in module order."""
    layers: dict[int, MoE] = {}
    for part in model_parts:
        for module in part.modules():
            if isinstance(module, MoE):
                layers.setdefault(id(module), module)
    return list(layers.values())


@torch.no_grad()
def reset_routing_statistics(model_parts: Sequence[nn.Module]) -> None:
    """Discard the observations of a step that never reached the optimizer hooks; the
    learned router weights and the persistent bias stay (bias_update.py:36-51)."""
    for moe in collect_moe_layers(model_parts):
        moe.tokens_per_expert_E.zero_()
        if isinstance(moe.router, QuantileBalancedTopKRouter):
            moe.router.quantile_balancer.required_bias_histogram_EB.zero_()


@torch.no_grad()
def collect_routing_load_metrics(model_parts: Sequence[nn.Module], parallel_dims=None,
                                 device: torch.device | None = None) -> dict[str, float]:
    """Load-balance observability from the token counters, read before the optimizer hooks
    drain them (bias_update.py:100-137): fraction of empty experts, coefficient of variation
    and max-to-mean load, averaged (max: maximised) over the blocks that saw tokens.  A few
    ``(E,)`` reductions and one host read-back per call; a logging path, not a hot one."""
    _single_process(parallel_dims)
    layers = collect_moe_layers(model_parts)
    if not layers:
        return {}
    device = device if device is not None else layers[0].tokens_per_expert_E.device
    totals = torch.zeros(4, device=device, dtype=torch.float32)
    for values in {id(m.tokens_per_expert_E): m.tokens_per_expert_E for m in layers}.values():
        values = values.to(device).float()
        mean = values.mean()
        active = (mean > 0).float()
        denominator = mean.clamp_min(1e-12)
        totals[0] += active
        totals[1] += active * (values == 0).float().mean()
        totals[2] += active * values.std(unbiased=False) / denominator
        totals[3] = torch.maximum(totals[3], active * values.max() / denominator)
    count, empty, cv, maximum = totals.tolist()
    if not count:
        return {}
    return {
        "moe/empty_expert_fraction": empty / count,
        "moe/load_cv": cv / count,
        "moe/max_to_mean_load": maximum,
    }


def _unique(moe_layers: Sequence[MoE]) -> list[MoE]:
    return list({id(moe): moe for moe in moe_layers}.values())


@torch.no_grad()
def update_expert_bias(moe_layers: Sequence[MoE], *, parallel_dims=None) -> None:
    """Sign-based update of every block from its accumulated counts (bias_update.py:140-195).
    Blocks that share one bias buffer are updated once, from their summed counts."""
    _single_process(parallel_dims)
    unique_layers = _unique(moe_layers)
    groups: dict[int, list[MoE]] = {}
    for moe in unique_layers:
        key = id(moe.expert_bias_E) if moe.expert_bias_E is not None else id(moe)
        groups.setdefault(key, []).append(moe)
    for members in groups.values():
        if any(m.load_balance_coeff != members[0].load_balance_coeff for m in members):
            raise ValueError("Shared expert bias requires identical load_balance_coeff")
    for members in groups.values():
        owner = members[0]
        for other in members[1:]:
            owner.tokens_per_expert_E.add_(other.tokens_per_expert_E)
        owner.update_expert_bias()
        if owner.load_balance_coeff is not None and owner.expert_bias_E is not None:
            for other in members[1:]:
                other.tokens_per_expert_E.zero_()


@torch.no_grad()
def update_quantile_expert_bias(moe_layers: Sequence[MoE], *, parallel_dims=None) -> None:
    """Write every block's next bias from its histogram, then drain histogram and token
    counter for the next accumulation window (bias_update.py:198-246)."""
    _single_process(parallel_dims)
    unique_layers = _unique(moe_layers)
    groups: dict[int, list[MoE]] = {}
    for moe in unique_layers:
        groups.setdefault(id(moe.expert_bias_E), []).append(moe)
    for members in groups.values():
        owner = members[0].router.quantile_balancer
        policy = (owner.num_experts, owner.top_k, owner.num_bins)
        for other in members[1:]:
            b = other.router.quantile_balancer
            if (b.num_experts, b.top_k, b.num_bins) != policy:
                raise ValueError("Shared quantile bias requires identical histogram policy")
    for members in groups.values():
        owner = members[0]
        combined = owner.router.quantile_balancer.required_bias_histogram_EB
        if len(members) > 1:
            combined = combined.clone()
            for other in members[1:]:
                combined.add_(other.router.quantile_balancer.required_bias_histogram_EB)
        owner.expert_bias_E.copy_(
            owner.router.quantile_balancer.estimate_expert_bias(combined, owner.expert_bias_E)
        )
        for moe in members:
            moe.router.quantile_balancer.required_bias_histogram_EB.zero_()
            moe.tokens_per_expert_E.zero_()


def register_moe_balancing_hook(optimizer: torch.optim.Optimizer, *, model_parts: Sequence[nn.Module],
                                parallel_dims=None) -> None:
    """Validate one balancing policy for the whole model and register its optimizer step
    pre-hook (bias_update.py:249-288).  Dense models and models without balancing get no hook."""
    _single_process(parallel_dims)
    layers = collect_moe_layers(model_parts)
    if not layers:
        return
    quantile_count = sum(isinstance(moe.router, QuantileBalancedTopKRouter) for moe in layers)
    if quantile_count:
        if quantile_count != len(layers) or any(moe.load_balance_coeff is not None for moe in layers):
            raise ValueError(
                "Quantile-balanced routing is mutually exclusive with the "
                "sign-based load-balancing bias: every MoE layer must use a "
                "QuantileBalancedTopKRouter with load_balance_coeff=None, or "
                "none may."
            )
        update_bias = update_quantile_expert_bias
    else:
        enabled = layers[0].load_balance_coeff is not None
        if any((moe.load_balance_coeff is not None) != enabled for moe in layers):
            raise ValueError(
                "MoE load_balance_coeff must be configured consistently across "
                "all MoE layers. Either set it for every MoE layer or leave it "
                "unset for all MoE layers."
            )
        if not enabled:
            return
        update_bias = update_expert_bias
    optimizer.register_step_pre_hook(lambda *args, **kwargs: update_bias(layers))
