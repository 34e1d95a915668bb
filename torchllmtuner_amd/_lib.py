"""Loaders of the two shared libraries: ``libmi355moe.so`` (the HIP kernels behind the C
ABI declared in include/mi355_moe.h, bound here with ctypes) and ``libmi355moe_torch.so``
(their torch.library registration, the ``mi355_moe`` operator namespace).

The libraries are the only implementation of the MoE hot path: if one is missing or lacks
a symbol the import of the ops fails loudly -- there is no eager PyTorch or CPU fallback
behind them.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmi355moe.so")
TORCH_EXT_PATH = os.path.join(_HERE, "libmi355moe_torch.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

P = c_void_p
I = c_int
L = c_int64
F = c_float

# name -> (restype, argtypes); mirrors include/mi355_moe.h declaration by declaration
SIGNATURES = {
    "mi355_moe_abi_version": (I, []),
    "mi355_moe_last_error": (c_char_p, []),
    "mi355_router_gate_fwd_workspace_bytes": (L, [L, L, L]),
    "mi355_router_gate_fwd": (I, [P, I, P, I, P, P, P, L, L, L, P]),
    "mi355_router_gate_bwd_workspace_bytes": (L, [L, L, L]),
    "mi355_router_gate_bwd": (I, [P, P, I, P, I, P, P, P, L, L, L, P]),
    "mi355_balance_loss_workspace_bytes": (L, [L, L]),
    "mi355_balance_loss_fwd": (I, [P, P, P, P, P, P, L, L, P]),
    "mi355_balance_loss_bwd": (I, [P, P, P, P, P, L, L, P]),
    "mi355_router_select_fwd": (I, [P, P, P, P, P, P, L, L, L, I, I, F, I, I, I, P]),
    "mi355_router_select_cutoff_fwd": (I, [P, P, P, P, P, P, L, L, L, I, I, F, P]),
    "mi355_quantile_observe": (I, [P, P, P, P, P, L, L, L, P]),
    "mi355_quantile_estimate": (I, [P, P, P, P, L, L, L, P]),
    "mi355_router_select_bwd": (I, [P, P, P, P, P, L, L, L, I, I, F, I, P]),
    "mi355_rms_norm_fwd": (I, [P, P, I, P, P, L, L, F, P]),
    "mi355_rms_norm_bwd_workspace_bytes": (L, [L, L]),
    "mi355_rms_norm_bwd": (I, [P, P, P, P, I, P, P, P, L, L, P]),
    "mi355_permute_plan_workspace_bytes": (L, [L, L, L]),
    "mi355_permute_plan": (I, [P, L, L, L, L, L, L, L, P, P, P, P, P, P, L, P, P, P, L, P, P]),
    "mi355_segments_from_counts": (I, [P, L, L, L, P, P, P, P, P, L, P]),
    "mi355_permute_plan_static_max_bytes": (L, []),
    "mi355_permute_plan_static": (I, [P, L, L, L, L, L, L, L, P, P, P, P, P, P, L, P, P, P, L, P]),
    "mi355_permute_rows_fwd": (I, [P, I, P, P, P, P, L, L, L, L, P]),
    "mi355_permute_rows_bwd": (I, [P, I, P, P, L, L, L, P]),
    "mi355_combine_fwd": (I, [P, I, P, P, P, L, L, L, I, P]),
    "mi355_combine_bwd": (I, [P, P, I, P, P, P, P, P, P, L, L, L, L, P]),
    "mi355_grouped_tile_m": (L, [I]),
    "mi355_grouped_swiglu_fwd": (I, [P, P, L, P, P, P, I, P, P, P, P, P, L, P, P, P, P, L, L, L, L, P]),
    "mi355_grouped_swiglu_stage": (
        I,
        [I, P, P, P, L, P, P, P, P, P, P, P, P, P, P, P, P, L, P, P, P, P, P, P, L, L, L, L, P],
    ),
    "mi355_grouped_linear_fwd": (I, [P, P, I, P, P, P, P, P, L, P, L, L, L, L, P]),
    "mi355_grouped_linear_bwd": (I, [P, P, P, I, P, P, P, P, P, L, P, P, L, L, L, L, P]),
    "mi355_grouped_combine_bwd_slots": (L, [I, L, L]),
    "mi355_grouped_swiglu_combine_bwd": (
        I,
        [P, P, P, L, P, P, P, P, P, P, I, P, P, P, P, P, L, P, P, P, P, P, P, P, P, L, L, L, L, I, P],
    ),
    "mi355_combine_row_scale": (I, [P, P, P, L, L, L, P]),
    "mi355_combine_scores_bwd": (I, [P, L, P, P, L, L, L, P]),
    "mi355_grouped_swiglu_bwd": (
        I,
        [P, P, P, L, P, P, P, P, P, P, I, P, P, P, P, P, L, P, P, P, P, P, P, L, L, L, L, P],
    ),
}

ABI_VERSION = 3  # MI355_MOE_ABI_VERSION of include/mi355_moe.h

_lib = None


class MI355LibraryError(RuntimeError):
    """The HIP library is missing, stale or failed a call."""


def load():
    """Load the shared library once and attach the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise MI355LibraryError(
            f"{LIB_PATH} is not built. Run `make -C {CSRC_DIR}` (or "
            "`python -c 'import __graft_entry__ as g; g.build()'`); the MoE block has no "
            "fallback implementation."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        try:
            fn = getattr(lib, name)
        except AttributeError as exc:
            raise MI355LibraryError(f"{LIB_PATH} does not export {name}; rebuild it") from exc
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mi355_moe_abi_version() != ABI_VERSION:
        raise MI355LibraryError("libmi355moe.so ABI version mismatch; rebuild it")
    _lib = lib
    return lib


_torch_ops_loaded = False


def load_torch_ops() -> None:
    """Register the ``mi355_moe`` operators with PyTorch's dispatcher (once per process)."""
    global _torch_ops_loaded
    if _torch_ops_loaded:
        return
    load()  # the C ABI library first: the extension links against it
    if not os.path.exists(TORCH_EXT_PATH):
        raise MI355LibraryError(
            f"{TORCH_EXT_PATH} is not built. Run `make -C {CSRC_DIR}` (or "
            "`python -c 'import __graft_entry__ as g; g.build()'`); the MoE block has no "
            "fallback implementation."
        )
    import torch

    torch.ops.load_library(TORCH_EXT_PATH)
    if not hasattr(torch.ops.mi355_moe, "gather_experts_combine_fwd"):
        raise MI355LibraryError(f"{TORCH_EXT_PATH} did not register the mi355_moe operators; rebuild it")
    _torch_ops_loaded = True


def check(rc: int, what: str) -> None:
    if rc != 0:
        msg = load().mi355_moe_last_error().decode(errors="replace")
        err = ValueError if rc == -1 else MI355LibraryError
        raise err(f"{what} failed ({rc}): {msg}")
