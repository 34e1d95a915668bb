"""The native MoE block (router, dispatchers, grouped experts) on MI355X kernels."""

from .activation import SwiGLU
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
    "DenseSwiGLU",
    "DispatchObservation",
    "ExpertErrorCapture",
    "GroupedExperts",
    "LocalDispatchMetadata",
    "LocalShareTokenDispatcher",
    "LocalTokenDispatcher",
    "MoE",
    "PaddedTokenDispatcher",
    "RoutedExperts",
    "RouterGateLinear",
    "SwiGLU",
    "TokenChoiceTopKRouter",
]
