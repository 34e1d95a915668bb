"""The native MoE block (router, dispatchers, grouped experts) on MI355X kernels."""

from .activation import SwiGLU
from .auxiliary_loss import AuxLoss, MicrobatchWiseLoadBalanceLoss
from .experts import DenseSwiGLU, DispatchObservation, ExpertErrorCapture, GroupedExperts, RoutedExperts
from .layer import MoE
from .linear import RouterGateLinear
from .routing import TokenChoiceTopKRouter
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
    "RoutedExperts",
    "RouterGateLinear",
    "SwiGLU",
    "TokenChoiceTopKRouter",
]
