"""The native MoE block (router, dispatchers, grouped experts) on MI355X kernels."""

from .activation import ActivationFn, SituGLU, SwiGLU
from .auxiliary_loss import AuxLoss, MicrobatchWiseLoadBalanceLoss
from .bias_update import (
    collect_moe_layers,
    collect_routing_load_metrics,
    register_moe_balancing_hook,
    reset_routing_statistics,
    update_expert_bias,
    update_quantile_expert_bias,
)
from .convert import (
    convert_block,
    hf_expert_state_to_native,
    moe_from_packed_experts,
    native_ep_expert_key,
    native_expert_state_to_hf,
)
from .experts import DenseSwiGLU, DispatchObservation, ExpertErrorCapture, GroupedExperts, RoutedExperts
from .layer import MoE
from .linear import RouterGateLinear
from .routing import QuantileBalancedTopKRouter, QuantileBalancer, TokenChoiceTopKRouter
from .token_dispatch import (
    LocalDispatchMetadata,
    LocalShareTokenDispatcher,
    LocalTokenDispatcher,
    PaddedTokenDispatcher,
)

__all__ = [
    "AuxLoss",
    "DenseSwiGLU",
    "DispatchObservation",
    "ExpertErrorCapture",
    "GroupedExperts",
    "LocalDispatchMetadata",
    "LocalShareTokenDispatcher",
    "LocalTokenDispatcher",
    "MicrobatchWiseLoadBalanceLoss",
    "MoE",
    "PaddedTokenDispatcher",
    "QuantileBalancedTopKRouter",
    "QuantileBalancer",
    "RoutedExperts",
    "RouterGateLinear",
    "ActivationFn",
    "SituGLU",
    "SwiGLU",
    "TokenChoiceTopKRouter",
    "collect_moe_layers",
    "convert_block",
    "collect_routing_load_metrics",
    "hf_expert_state_to_native",
    "moe_from_packed_experts",
    "native_ep_expert_key",
    "native_expert_state_to_hf",
    "register_moe_balancing_hook",
    "reset_routing_statistics",
    "update_expert_bias",
    "update_quantile_expert_bias",
]
