"""MI355X-native MoE block behind TorchLLMTuner's native-MoE interface.

``torchllmtuner_amd.moe`` mirrors the reference's module classes; ``ops`` are the
tensor-level calls into ``libmi355moe.so`` (C ABI in ``include/mi355_moe.h``).
"""

from . import _lib, kernel_registry, moe, ops  # noqa: F401
from .moe import (  # noqa: F401
    DenseSwiGLU,
    GroupedExperts,
    LocalShareTokenDispatcher,
    LocalTokenDispatcher,
    MoE,
    PaddedTokenDispatcher,
    RoutedExperts,
    RouterGateLinear,
    SituGLU,
    SwiGLU,
    TokenChoiceTopKRouter,
)

__version__ = "0.1.0"
