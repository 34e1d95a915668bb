"""Kernel-registry seam: ``moe_token_permute`` and ``rms_norm`` served by the MI355X kernels.

The reference routes a handful of operators through a name -> {device type -> callable}
registry (``llmtuner/kernel/registry.py:22-103``) and exposes the MoE row gather as
``moe_token_permute(hidden_states, expert_ids, *, use_eager=False)``
(``llmtuner/kernel/ops/moe.py:10-28``) with a torch backend for ``"cpu"``
(``llmtuner/kernel/cpu/basic.py:48-56``) and a vendor backend for ``"npu"``
(``llmtuner/kernel/npu/basic.py:62-69``).  This module holds the same three registry
functions with the same argument meaning and error behaviour, and registers one backend,
``"cuda"`` (the device type PyTorch-ROCm reports for an MI355X), built on the permutation
plan and row-gather kernels.  It is also the function a maintainer registers into the
reference's own registry::

    from llmtuner.kernel import register_kernel
    from torchllmtuner_amd.kernel_registry import moe_token_permute_mi355
    register_kernel("moe_token_permute", "cuda")(moe_token_permute_mi355)
    register_kernel("rms_norm", "cuda")(rms_norm_mi355)

``rms_norm`` (``llmtuner/kernel/ops/rms_norm.py:10-31``) is the norm the decoder layer applies
right before the MoE block; it gets a ``"cuda"`` backend the same way.

There is no torch-math backend here: asking for one (``use_eager=True``, a CPU tensor,
``fallback_to_cpu=True`` with nothing registered for ``"cpu"``) raises.
"""

from __future__ import annotations

import logging
import math
from collections.abc import Callable
from typing import Any, TypeVar

import torch

from . import ops as F
from . import ops

logger = logging.getLogger(__name__)

Kernel = Callable[..., Any]
KernelFunction = TypeVar("KernelFunction", bound=Kernel)

_KERNEL_REGISTRY: dict[str, dict[str, Kernel]] = {}
_warned_fallbacks: set[tuple[str, str]] = set()

#: device type used when a call carries no tensor and names no device
default_device_type = "cuda"


def register_kernel(name: str, device_type: str) -> Callable[[KernelFunction], KernelFunction]:
    """Decorator that binds ``function`` to ``(name, device_type)``.

    Follows ``registry.py:22-46``: empty or non-string identifiers raise ``ValueError``
    ("must not be empty"), a non-callable raises ``TypeError`` ("callable"), registering
    the same function twice is a no-op, a different function for a taken slot raises
    ``ValueError`` ("already registered").
    """
    for ident in (name, device_type):
        if not isinstance(ident, str) or not ident.strip():
            raise ValueError("Kernel name and device type must not be empty")

    def bind(function: KernelFunction) -> KernelFunction:
        if not callable(function):
            raise TypeError("Kernel implementation must be callable")
        slot = _KERNEL_REGISTRY.setdefault(name, {})
        taken = slot.get(device_type)
        if taken is not None and taken is not function:
            raise ValueError(f"Kernel {name!r} already registered for {device_type!r}")
        slot[device_type] = function
        return function

    return bind


def get_kernel(name: str, device_type: str | None = None, *, fallback_to_cpu: bool = False) -> Kernel:
    """Look up a backend (``registry.py:49-76``): ``KeyError`` "not registered" for an
    unknown name, "not available" for an unknown device; the ``"cpu"`` backend is used
    instead only on request, only if one is registered, with one warning per pair."""
    if device_type is None:
        device_type = default_device_type
    try:
        slot = _KERNEL_REGISTRY[name]
    except KeyError:
        raise KeyError(f"Kernel {name!r} is not registered") from None
    if device_type in slot:
        return slot[device_type]
    if fallback_to_cpu and "cpu" in slot:
        if (name, device_type) not in _warned_fallbacks:
            _warned_fallbacks.add((name, device_type))
            logger.warning(
                "Kernel %s is unavailable on %s; using the torch reference "
                "implementation without moving tensors", name, device_type)
        return slot["cpu"]
    raise KeyError(f"Kernel {name!r} is not available for device {device_type!r}")


def dispatch_kernel(name: str, *args: Any, device_type: str | None = None,
                    fallback_to_cpu: bool = False, **kwargs: Any) -> Any:
    """Pick the backend from the first tensor argument's device unless ``device_type``
    is given, then call it (``registry.py:79-103``).  Tensors are never moved."""
    if device_type is None:
        for value in (*args, *kwargs.values()):
            if isinstance(value, torch.Tensor):
                device_type = value.device.type
                break
    return get_kernel(name, device_type, fallback_to_cpu=fallback_to_cpu)(*args, **kwargs)


def _check_permutation_inputs(hidden_states: torch.Tensor, expert_ids: torch.Tensor) -> None:
    """Metadata-only validation, ``llmtuner/kernel/validation.py:123-133``."""
    if hidden_states.device != expert_ids.device:
        raise ValueError(
            f"Kernel inputs must share a device, got {hidden_states.device} and {expert_ids.device}")
    if hidden_states.ndim != 2 or expert_ids.ndim != 2:
        raise ValueError("MoE permutation expects [tokens, hidden] and [tokens, top_k]")
    if expert_ids.dtype not in (torch.int32, torch.int64):
        raise ValueError("MoE expert IDs must use int32 or int64")
    if expert_ids.shape[0] != hidden_states.shape[0] or expert_ids.shape[1] == 0:
        raise ValueError("MoE token counts must match and top_k must be positive")


@register_kernel("moe_token_permute", "cuda")
def moe_token_permute_mi355(hidden_states: torch.Tensor, expert_ids: torch.Tensor, *,
                            num_experts: int | None = None) -> torch.Tensor:
    """``hidden_states[argsort(expert_ids.flatten(), stable=True) // top_k]`` on the GPU.

    Returns ``[tokens * top_k, hidden]`` rows in stable expert-major order; gradients sum
    into the token rows (the row-gather backward kernel, no atomics).  The interface does
    not carry the number of experts; without ``num_experts`` it is read back from
    ``expert_ids.max()`` (one host synchronisation), so callers on a hot path pass it.
    """
    _check_permutation_inputs(hidden_states, expert_ids)
    if hidden_states.device.type != "cuda":
        raise RuntimeError(
            f"moe_token_permute_mi355 needs tensors on a HIP device, got {hidden_states.device}")
    if hidden_states.shape[0] == 0:
        return hidden_states[:0]
    if num_experts is None:
        lo, hi = (int(v) for v in torch.aminmax(expert_ids))
        if lo < 0:
            raise ValueError(f"MoE expert IDs must be non-negative, got {lo}")
        num_experts = hi + 1
    plan = ops.permute_plan(expert_ids, num_experts)
    return F.permute_rows(hidden_states, plan)


def moe_token_permute(hidden_states: torch.Tensor, expert_ids: torch.Tensor, *,
                      use_eager: bool = False, num_experts: int | None = None) -> torch.Tensor:
    """The reference operator (``kernel/ops/moe.py:10-28``), dispatched on the input's
    device.  ``use_eager`` asks for torch math, which this package does not carry."""
    if use_eager:
        raise NotImplementedError(
            "moe_token_permute: no torch-math backend in this package; the HIP kernel is "
            "the only implementation")
    extra = {} if num_experts is None else {"num_experts": num_experts}
    return dispatch_kernel("moe_token_permute", hidden_states, expert_ids, **extra)


def _check_rms_norm_inputs(hidden_states: torch.Tensor, weight: torch.Tensor, epsilon: float) -> None:
    """Metadata-only validation, ``llmtuner/kernel/validation.py:110-120``."""
    if hidden_states.device != weight.device:
        raise ValueError(f"Kernel inputs must share a device, got {hidden_states.device} and {weight.device}")
    if weight.ndim != 1 or hidden_states.ndim == 0:
        raise ValueError("RMSNorm requires a 1-D weight and a non-scalar input")
    if hidden_states.shape[-1] != weight.shape[0] or weight.numel() == 0:
        raise ValueError("RMSNorm weight must match the nonzero final input dimension")
    if not math.isfinite(epsilon) or epsilon < 0:
        raise ValueError("RMSNorm epsilon must be finite and nonnegative")


@register_kernel("rms_norm", "cuda")
def rms_norm_mi355(hidden_states: torch.Tensor, weight: torch.Tensor, epsilon: float) -> torch.Tensor:
    """``hidden_states * rsqrt(mean(hidden_states**2, -1) + epsilon) * weight`` on the GPU,
    computed in fp32 and rounded once to the input dtype (what
    ``torch.nn.functional.rms_norm``, the reference's CPU backend, returns); differentiable
    in both arguments.  Input and weight share a dtype (fp32 or bf16), as the reference
    leaves dtype conversion to the caller."""
    _check_rms_norm_inputs(hidden_states, weight, epsilon)
    if hidden_states.device.type != "cuda":
        raise RuntimeError(f"rms_norm_mi355 needs tensors on a HIP device, got {hidden_states.device}")
    return F.rms_norm(hidden_states, weight, epsilon)


def rms_norm(hidden_states: torch.Tensor, weight: torch.Tensor, epsilon: float, *,
             use_eager: bool = False) -> torch.Tensor:
    """The public operator of ``llmtuner/kernel/ops/rms_norm.py:10-31``, dispatched on the
    input's device.  ``use_eager`` asks for torch math, which this package does not carry."""
    if use_eager:
        raise NotImplementedError(
            "rms_norm: no torch-math backend in this package; the HIP kernel is the only implementation")
    return dispatch_kernel("rms_norm", hidden_states, weight, epsilon)


__all__ = [
    "dispatch_kernel",
    "get_kernel",
    "moe_token_permute",
    "moe_token_permute_mi355",
    "register_kernel",
    "rms_norm",
    "rms_norm_mi355",
]
