"""Tensor-level entry points of the MoE kernels: the ``mi355_moe`` torch.library operators.

``libmi355moe_torch.so`` registers one operator per stage (``torch.ops.mi355_moe.*``): a
thin C++ layer that allocates outputs with PyTorch's allocator and calls the C ABI of
``include/mi355_moe.h`` on the current HIP stream.  This module adds what the dispatcher
needs around them -- shape propagation for fake / meta tensors (so the operators trace
under ``torch.compile``; the autograd formulas are C++ nodes inside ``libmi355moe_torch.so`` whose
backward passes are again operators of the same library) -- plus Python wrappers that validate arguments the way the
reference's modules do and carry the permutation plan as one object.

Every function requires device tensors and raises if given CPU tensors: the kernels are the
only implementation.  The profiling hooks at the end (one MFMA kernel per call on
pre-allocated buffers) go straight to the C ABI through ``ctypes``.
"""

from __future__ import annotations

import atexit
import time
from dataclasses import dataclass

import torch

from . import _lib

_lib.load_torch_ops()  # fails loudly when the library is not built
_O = torch.ops.mi355_moe

_DT = {torch.float32: 0, torch.bfloat16: 1, torch.float64: 2}
SCORE_FUNCS = {"sigmoid": 0, "softmax": 1, "sqrtsoftplus": 2}
SELECT_TOPK, SELECT_FIXED, SELECT_BALANCED = 0, 1, 2
# most rows an entry of a plan's tile list covers: the library's row-tile height
TILE_M = int(_lib.load().mi355_grouped_tile_m(_DT[torch.bfloat16]))


def _dt(t: torch.Tensor, fp64: bool = True) -> int:
    """The library's code for the tensor's dtype.  fp64 passes through the router gate (converted
    to fp32 on the way in, as the reference does), the row movers, the combine and the grouped
    experts (fp64 arithmetic throughout); ``fp64=False`` is for the kernels that have no fp64 form."""
    code = _DT.get(t.dtype)
    if code is None or (code == 2 and not fp64):
        raise TypeError(f"MI355 MoE kernels support float32 and bfloat16{' (and float64)' if fp64 else ''}, got {t.dtype}")
    return code


def _dev(*tensors: torch.Tensor | None) -> torch.device:
    dev = None
    for t in tensors:
        if t is None:
            continue
        if t.device.type != "cuda":
            raise RuntimeError(
                "MI355 MoE kernels need tensors on a HIP device (got "
                f"{t.device}); there is no CPU implementation"
            )
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise RuntimeError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def _p(t: torch.Tensor | None):
    return None if t is None else t.data_ptr()


def _stream(dev: torch.device):
    return torch.cuda.current_stream(dev).cuda_stream


def tile_m(dtype: torch.dtype = torch.bfloat16) -> int:
    return TILE_M


def _opt(t: torch.Tensor, wanted: bool):
    """Operators return an empty (0,) tensor for an output that was not asked for."""
    return t if wanted else None


_AUX_STREAMS: dict = {}


def aux_stream(device: torch.device):
    """The library's stream for work that may run beside the current stream of ``device`` (the
    shared expert of a block), as a ``torch.cuda.ExternalStream`` of default priority, or None
    when there is none: it is created on the first call that is not under stream capture."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    stream = _AUX_STREAMS.get(index)
    if stream is None:
        address = _O.aux_stream(index)
        if not address:
            return None
        stream = _AUX_STREAMS[index] = torch.cuda.ExternalStream(address, device=torch.device("cuda", index))
    return stream


def _let_autograd_threads_finish():
    """Runs at interpreter exit.  After a backward pass the autograd engine's device thread may still be
    releasing that pass's results; for the ones Python holds a wrapper of it needs the GIL, and CPython
    ends a thread that asks for the GIL once finalisation has begun, which aborts the process (status
    134, after all work is done) when the script exits within milliseconds of its last backward pass.
    Giving up the GIL for a moment before finalisation begins lets that thread finish."""
    if torch.cuda.is_initialized():
        time.sleep(0.05)


atexit.register(_let_autograd_threads_finish)


# ====================================================================== fake kernels
# Shape / dtype propagation for tracing.  Skipped outputs are empty (0,) tensors.
def _fake(name):
    return torch.library.register_fake(f"mi355_moe::{name}")


def _e0(like, dtype=None):
    return like.new_empty((0,), dtype=dtype or like.dtype)


@_fake("router_gate_fwd")
def _(x, w, logit_bias):
    return x.new_empty((x.shape[0], w.shape[0]), dtype=torch.float32)


@_fake("router_gate_bwd")
def _(dlogits, x, w, need_dx, need_dw):
    return (torch.empty_like(x) if need_dx else _e0(x)), (torch.empty_like(w) if need_dw else _e0(w))


@_fake("router_select_fwd")
def _(logits, expert_bias, top_k, score_func, route_norm, route_scale, num_groups, num_limited, mode,
      want_scores, want_map):
    T, E = logits.shape
    return (logits.new_empty((T, top_k)), logits.new_empty((T, top_k), dtype=torch.int64),
            logits.new_empty((T, E)) if want_scores else _e0(logits),
            logits.new_empty((T, E) if want_map else (0, 0), dtype=torch.bool))


@_fake("router_select_cutoff_fwd")
def _(logits, expert_bias, top_k, score_func, route_norm, route_scale):
    T, E = logits.shape
    return (logits.new_empty((T, top_k)), logits.new_empty((T, top_k), dtype=torch.int64),
            logits.new_empty((T, E)), logits.new_empty((T,)))


@_fake("router_select_bwd")
def _(logits, ids, dweights, dscores, score_func, route_norm, route_scale, mode):
    return torch.empty_like(logits)


@_fake("quantile_observe")
def _(histogram, scores, cutoff, expert_bias, padding_mask):
    return None


@_fake("quantile_estimate")
def _(histogram, expert_bias, top_k):
    return expert_bias.new_empty((histogram.shape[0],), dtype=torch.float32)


@_fake("rms_norm_fwd")
def _(x, weight, epsilon):
    rows = x.numel() // max(weight.numel(), 1)
    return torch.empty_like(x), x.new_empty((rows,), dtype=torch.float32)


@_fake("rms_norm_bwd")
def _(dy, x, weight, rstd, need_dx, need_dw):
    return (torch.empty_like(x) if need_dx else _e0(x)), (torch.empty_like(weight) if need_dw else _e0(weight))


@_fake("balance_loss_fwd")
def _(scores, routing_map, padding_mask):
    return scores.new_empty((1 + scores.shape[1],))


@_fake("balance_loss_bwd")
def _(scores, f, padding_mask, grad_loss):
    return torch.empty_like(scores)


def _plan_sizes(N, El, align):
    row_cap = N + (El * (align - 1) if align > 1 else 0)
    tile_cap = N // TILE_M + El + 1
    return row_cap, tile_cap


@_fake("permute_plan")
def _(ids, num_experts, local_lo, local_hi, align):
    T, K = ids.shape
    El = local_hi - local_lo
    row_cap, tile_cap = _plan_sizes(T * K, El, align)
    i32 = dict(dtype=torch.int32)
    return (ids.new_empty((num_experts + (El + 1) + 2 * El + 2 * tile_cap + 1,), **i32),
            ids.new_empty((T * K,), **i32), ids.new_empty((2, row_cap), **i32))


@_fake("segments_from_counts")
def _(counts, total_rows):
    El = counts.shape[0]
    tile_cap = total_rows // TILE_M + El + 1
    return counts.new_empty(((El + 1) + 2 * El + 2 * tile_cap + 1,), dtype=torch.int32)


@_fake("permute_rows_fwd")
def _(x, row_of_slot, slot_of_row, total_rows, top_k, row_capacity):
    return x.new_empty((row_capacity, x.shape[1]))


@_fake("permute_rows_bwd")
def _(drows, row_of_slot, num_tokens, top_k):
    return drows.new_empty((num_tokens, drows.shape[1]))


@_fake("combine_fwd")
def _(y, weights, row_of_slot, slot_of_row, total_rows, num_tokens, top_k, round_terms):
    return y.new_empty((num_tokens, y.shape[1]))


@_fake("combine_bwd")
def _(dout, y, weights, row_of_slot, slot_of_row, total_rows, top_k):
    return torch.empty_like(y), y.new_empty((dout.shape[0], top_k), dtype=torch.float32)


@_fake("combine_row_scale")
def _(weights, slot_of_row, row_capacity):
    return weights.new_empty((row_capacity,), dtype=torch.float32)


@_fake("combine_scores_bwd")
def _(dot_partial, row_of_slot, num_tokens, top_k):
    return dot_partial.new_empty((num_tokens, top_k))


@_fake("grouped_swiglu_fwd")
def _(rows, token_of_row, w1, w3, w2, seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles,
      row_capacity, zero_fill):
    F, D = w1.shape[1], rows.shape[1]
    mk = lambda n: rows.new_empty((row_capacity, n))
    return mk(D), mk(F), mk(F), mk(F)


@_fake("grouped_swiglu_bwd")
def _(dy, rows, token_of_row, w1, w3, w2, gate, up, h, seg_offsets, seg_counts, tile_expert, tile_row0,
      num_tiles, need_drows, need_dw, zero_fill):
    drows = rows.new_empty((dy.shape[0], rows.shape[1])) if need_drows else _e0(rows)
    g = lambda w: torch.empty_like(w) if need_dw else _e0(w)
    return drows, g(w1), g(w3), g(w2)


@_fake("grouped_linear_fwd")
def _(x, w, seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, zero_fill):
    return x.new_empty((x.shape[0], w.shape[1]))


@_fake("grouped_linear_bwd")
def _(dy, x, w, seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, need_dx, need_dw, zero_fill):
    return (torch.empty_like(x) if need_dx else _e0(x)), (torch.empty_like(w) if need_dw else _e0(w))


@_fake("rows_experts_combine_fwd")
def _(x, weights, w1, w3, w2, row_of_slot, slot_of_row, total_rows, seg_offsets, seg_counts, tile_expert, tile_row0,
      num_tiles, top_k, row_capacity, round_terms):
    F = w1.shape[1]
    mk = lambda n: x.new_empty((row_capacity, n))
    return torch.empty_like(x), mk(x.shape[1]), mk(F), mk(F), mk(F), mk(x.shape[1])


@_fake("rows_experts_combine_bwd")
def _(dout, rows, weights, w1, w3, w2, gate, up, h, y, row_of_slot, slot_of_row, total_rows, seg_offsets, seg_counts,
      tile_expert, tile_row0, num_tiles, num_tokens, top_k, need_dx, need_dw):
    g = lambda w: torch.empty_like(w) if need_dw else _e0(w)
    dx = rows.new_empty((num_tokens, rows.shape[1])) if need_dx else _e0(rows)
    return dx, g(w1), g(w3), g(w2), rows.new_empty((num_tokens, top_k), dtype=torch.float32)


@_fake("gather_experts_combine_fwd")
def _(x, weights, w1, w3, w2, token_of_row, slot_of_row, row_of_slot, seg_offsets, seg_counts, tile_expert,
      tile_row0, num_tiles, top_k, row_capacity, round_terms, save_gate_up):
    F = w1.shape[1]
    rows = row_capacity if save_gate_up else 0
    return torch.empty_like(x), x.new_empty((rows, F)), x.new_empty((rows, F))


@_fake("gather_experts_combine_bwd")
def _(dout, x, weights, w1, w3, w2, gate, up, token_of_row, slot_of_row, row_of_slot, seg_offsets, seg_counts,
      tile_expert, tile_row0, num_tiles, top_k, need_dx, need_dw):
    g = lambda w: torch.empty_like(w) if need_dw else _e0(w)
    return ((torch.empty_like(x) if need_dx else _e0(x)), g(w1), g(w3), g(w2),
            x.new_empty((x.shape[0], top_k), dtype=torch.float32))


# ====================================================================== autograd formulas
# Each differentiable operator's backward is the hand-written kernel for that stage (linear.py:133-151 is
# the gate's formula).  The formulas are C++ autograd nodes registered for the operators' Autograd key in
# csrc/torch_autograd.cpp: they call the backward operators through the dispatcher, so the fake kernels
# above serve tracing in both directions, and they run on the engine's thread without the interpreter
# lock.


# ====================================================================== router
def router_gate_fwd(x_TD, w_ED, logit_bias_E=None):
    """fp32 logits (differentiable: dX in the input dtype, dW in the weight dtype)."""
    _dev(x_TD, w_ED, logit_bias_E)
    if w_ED.shape[1] != x_TD.shape[1]:
        raise ValueError(f"gate weight {tuple(w_ED.shape)} does not match input dim {x_TD.shape[1]}")
    _dt(x_TD), _dt(w_ED)
    return _O.router_gate_fwd(x_TD, w_ED, logit_bias_E)


def router_gate_bwd(dlogits_TE, x_TD, w_ED, need_dx=True, need_dw=True):
    _dev(dlogits_TE, x_TD, w_ED)
    dx, dw = _O.router_gate_bwd(dlogits_TE, x_TD, w_ED, bool(need_dx), bool(need_dw))
    return _opt(dx, need_dx), _opt(dw, need_dw)


def router_select_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                      num_groups=0, num_limited=0, mode=SELECT_TOPK, want_scores=False, want_map=False):
    """Returns ``(weights_TK, ids_TK, scores_TE or None)`` -- and the bool routing map as a
    fourth item when ``want_map`` is set.  Differentiable in the logits through the weights
    and (when materialised) the dense scores."""
    _dev(logits_TE, expert_bias_E)
    if logits_TE.dtype != torch.float32:
        raise TypeError("router logits must be float32")
    weights, ids, scores, rmap = _O.router_select_fwd(
        logits_TE, expert_bias_E, int(top_k), SCORE_FUNCS[score_func], bool(route_norm), float(route_scale),
        int(num_groups or 0), int(num_limited or 0), int(mode), bool(want_scores), bool(want_map))
    scores = scores if want_scores else None
    return (weights, ids, scores, rmap) if want_map else (weights, ids, scores)


def router_select_cutoff_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
    """Biased top-k plus the (K+1)-th biased score of every token: returns
    ``(weights_TK, ids_TK, scores_TE, cutoff_T)``."""
    _dev(logits_TE, expert_bias_E)
    if logits_TE.dtype != torch.float32:
        raise TypeError("router logits must be float32")
    return _O.router_select_cutoff_fwd(logits_TE, expert_bias_E, int(top_k), SCORE_FUNCS[score_func],
                                       bool(route_norm), float(route_scale))


def router_select_bwd(logits_TE, ids_TK, dweights_TK, dscores_TE, score_func, route_norm,
                      route_scale, mode=SELECT_TOPK):
    _dev(logits_TE, ids_TK, dweights_TK, dscores_TE)
    return _O.router_select_bwd(logits_TE, ids_TK, dweights_TK, dscores_TE, SCORE_FUNCS[score_func],
                                bool(route_norm), float(route_scale), int(mode))


def quantile_observe(histogram_EB, scores_TE, cutoff_T, expert_bias_E, padding_mask_T=None):
    """Accumulates the required-bias histogram in place (int64 ``(E, B)``)."""
    _dev(histogram_EB, scores_TE, cutoff_T, expert_bias_E, padding_mask_T)
    if histogram_EB.dtype != torch.int64 or not histogram_EB.is_contiguous():
        raise TypeError("histogram_EB must be a contiguous int64 tensor")
    T, E = scores_TE.shape
    if histogram_EB.shape[0] != E or cutoff_T.numel() != T or expert_bias_E.numel() != E:
        raise ValueError(
            f"quantile_observe: histogram {tuple(histogram_EB.shape)}, scores {(T, E)}, "
            f"cutoff {tuple(cutoff_T.shape)} and bias {tuple(expert_bias_E.shape)} do not agree"
        )
    pad = None
    if padding_mask_T is not None:
        if padding_mask_T.dtype != torch.bool or padding_mask_T.numel() != T:
            raise ValueError("padding_mask_T must be a bool tensor with one entry per token")
        pad = padding_mask_T.reshape(-1)
    _O.quantile_observe(histogram_EB, scores_TE, cutoff_T, expert_bias_E, pad)


def quantile_estimate(histogram_EB, expert_bias_E, top_k):
    """The next mean-centred expert bias (new tensor, dtype of ``expert_bias_E``)."""
    _dev(histogram_EB, expert_bias_E)
    if histogram_EB.dtype != torch.int64:
        raise TypeError("histogram_EB must be int64")
    return _O.quantile_estimate(histogram_EB, expert_bias_E, int(top_k)).to(expert_bias_E.dtype)


def rms_norm_fwd(x, weight, epsilon):
    """Returns ``(y, rstd)``; ``x`` is ``(..., D)``, ``weight`` ``(D,)`` of the same dtype.
    Differentiable through ``y``."""
    _dev(x, weight)
    if x.dtype != weight.dtype:
        raise TypeError(f"rms_norm: input ({x.dtype}) and weight ({weight.dtype}) must share a dtype")
    _dt(x, fp64=False)
    return _O.rms_norm_fwd(x, weight, float(epsilon))


def rms_norm_bwd(dy, x, weight, rstd, need_dx=True, need_dw=True):
    """Returns ``(dx or None, dweight or None)``."""
    _dev(dy, x, weight, rstd)
    dx, dw = _O.rms_norm_bwd(dy, x, weight, rstd, bool(need_dx), bool(need_dw))
    return _opt(dx, need_dx), _opt(dw, need_dw)


def _as_bool(m):
    return m if m.dtype == torch.bool else m.ne(0)


def balance_loss_fwd(scores_TE, routing_map_TE, padding_mask_T=None):
    """Returns (loss 0-d fp32, f_E) of the per-forward load-balance loss; the loss is
    differentiable in the scores."""
    _dev(scores_TE, routing_map_TE, padding_mask_T)
    if scores_TE.dtype != torch.float32:
        raise TypeError("router scores must be float32")
    if routing_map_TE.shape != scores_TE.shape:
        raise ValueError(f"routing map {tuple(routing_map_TE.shape)} does not match scores {tuple(scores_TE.shape)}")
    out = _O.balance_loss_fwd(scores_TE, _as_bool(routing_map_TE),
                              None if padding_mask_T is None else _as_bool(padding_mask_T))
    return out[0], out[1:]


def balance_loss_bwd(scores_TE, f_E, grad_loss, padding_mask_T=None):
    _dev(scores_TE, f_E, grad_loss, padding_mask_T)
    pad = None if padding_mask_T is None else _as_bool(padding_mask_T)
    return _O.balance_loss_bwd(scores_TE, f_E, pad, grad_loss)


# ====================================================================== plan
@dataclass
class PermutePlan:
    """Device-resident description of the expert-major row layout (all int32)."""

    num_tokens: int
    top_k: int
    num_experts: int
    local_lo: int
    local_hi: int
    align: int
    tile_m: int
    row_capacity: int
    tile_capacity: int
    counts_E: torch.Tensor | None
    seg_offsets: torch.Tensor
    seg_counts: torch.Tensor
    row_of_slot: torch.Tensor | None
    slot_of_row: torch.Tensor | None
    token_of_row: torch.Tensor | None
    tile_expert: torch.Tensor
    tile_row0: torch.Tensor
    num_tiles: torch.Tensor
    # local experts by descending row count; lives right behind seg_counts in memory, where
    # the weight-gradient kernels look for it
    expert_order: torch.Tensor | None = None

    @property
    def num_local_experts(self) -> int:
        return self.local_hi - self.local_lo

    @property
    def total_rows(self) -> torch.Tensor:
        """0-d device view of the number of rows in use (padding included)."""
        return self.seg_offsets[self.num_local_experts]

    def total_rows_1(self) -> torch.Tensor:
        """The same as a 1-element view (what the operators take)."""
        El = self.num_local_experts
        return self.seg_offsets[El:El + 1]

    def pad_index(self):
        """slot_of_row when the plan has padding rows (they must read as zeros), else None."""
        return self.slot_of_row if self.align > 1 else None

    def segments(self):
        return self.seg_offsets, self.seg_counts, self.tile_expert, self.tile_row0, self.num_tiles


def _split_small(small, E, El, tile_cap):
    # one call for the seven views (sliced one by one they cost a microsecond of host time each);
    # 2*El ints hold the counts, then the experts by descending count
    sizes = [E, El + 1, El, El, tile_cap, tile_cap, 1]
    counts_E, seg_offsets, seg_counts, expert_order, tile_expert, tile_row0, num_tiles = small[:sum(sizes)].split(sizes)
    return (counts_E if E else None), seg_offsets, seg_counts, expert_order, tile_expert, tile_row0, num_tiles


def permute_plan(ids_TK, num_experts, local_lo=0, local_hi=None, align=1) -> PermutePlan:
    _dev(ids_TK)
    T, K = ids_TK.shape
    E = int(num_experts)
    hi = E if local_hi is None else int(local_hi)
    lo = int(local_lo)
    El = hi - lo
    align = int(align)
    row_cap, tile_cap = _plan_sizes(T * K, El, align)
    small, row_of_slot, rows2 = _O.permute_plan(ids_TK, E, lo, hi, align)
    counts_E, seg_offsets, seg_counts, expert_order, tile_expert, tile_row0, num_tiles = _split_small(
        small, E, El, tile_cap)
    return PermutePlan(T, K, E, lo, hi, align, TILE_M, row_cap, tile_cap, counts_E, seg_offsets,
                       seg_counts, row_of_slot, rows2[0], rows2[1], tile_expert, tile_row0, num_tiles,
                       expert_order)


def segments_from_counts(counts_e, total_rows: int) -> PermutePlan:
    """Plan for rows that are already expert-major with ``counts_e`` rows each."""
    _dev(counts_e)
    El = counts_e.shape[0]
    tile_cap = total_rows // TILE_M + El + 1
    small = _O.segments_from_counts(counts_e, total_rows)
    _, seg_offsets, seg_counts, expert_order, tile_expert, tile_row0, num_tiles = _split_small(small, 0, El, tile_cap)
    return PermutePlan(0, 1, El, 0, El, 1, TILE_M, total_rows, tile_cap, None, seg_offsets, seg_counts,
                       None, None, None, tile_expert, tile_row0, num_tiles, expert_order)


# ====================================================================== row movers
def permute_rows_fwd(x_TD, plan: PermutePlan):
    """rows[r] = x[token of row r], zeros in padding rows.  Differentiable in ``x`` (the
    backward sums each token's K row gradients)."""
    _dev(x_TD, plan.row_of_slot)
    _dt(x_TD)
    return _O.permute_rows_fwd(x_TD, plan.row_of_slot, plan.pad_index(), plan.total_rows_1(), plan.top_k,
                               plan.row_capacity)


def permute_rows_bwd(drows_RD, plan: PermutePlan):
    _dev(drows_RD, plan.row_of_slot)
    return _O.permute_rows_bwd(drows_RD, plan.row_of_slot, plan.num_tokens, plan.top_k)


def combine_fwd(y_RD, weights_TK, plan: PermutePlan, round_terms=True):
    """out[t] = sum_k weights[t,k] * y[row(t,k)].  Differentiable in ``y`` and ``weights``."""
    _dev(y_RD, weights_TK, plan.row_of_slot)
    _dt(y_RD)
    return _O.combine_fwd(y_RD, weights_TK, plan.row_of_slot, plan.pad_index(), plan.total_rows_1(),
                          plan.num_tokens, plan.top_k, bool(round_terms))


def combine_bwd(dout_TD, y_RD, weights_TK, plan: PermutePlan, zero_padding=True):
    _dev(dout_TD, y_RD, weights_TK)
    pad = plan.pad_index() if zero_padding else None
    return _O.combine_bwd(dout_TD, y_RD, weights_TK, plan.row_of_slot, pad, plan.total_rows_1(), plan.top_k)


# ====================================================================== experts
def gather_supported(x_TD, hidden_dim: int) -> bool:
    """The fused token gather exists for the bf16 MFMA kernels (D, F multiples of 64, at
    least 384: the library's own condition for that path) and addresses its source with
    32-bit byte offsets."""
    D = x_TD.shape[-1]
    return (x_TD.dtype == torch.bfloat16 and D % 64 == 0 and hidden_dim % 64 == 0
            and D >= 384 and hidden_dim >= 384 and 1 <= x_TD.shape[0] and x_TD.shape[0] * D * 2 < 2**32)


def _check_experts(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan):
    D = rows_RD.shape[1]
    El, F, D2 = w1_EFD.shape
    if D2 != D or w3_EFD.shape != w1_EFD.shape or tuple(w2_EDF.shape) != (El, D, F):
        raise ValueError("expert weight shapes do not match (E,F,D)/(E,F,D)/(E,D,F)")
    if not (w1_EFD.dtype == w3_EFD.dtype == w2_EDF.dtype == rows_RD.dtype):
        raise TypeError("expert weights and rows must share one dtype")
    if El != plan.num_local_experts:
        raise ValueError(f"plan covers {plan.num_local_experts} experts, weights hold {El}")
    _dt(rows_RD)


def grouped_swiglu_fwd(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan: PermutePlan, gather=False, zero_fill=False):
    """Returns ``(y, gate, up, h)``; ``y`` is differentiable in the rows and the weights
    (not with ``gather``: that case is differentiated through ``gather_experts_combine``).

    ``gather=True``: ``rows_RD`` is the (T, D) token matrix, read through ``plan.token_of_row``.
    ``zero_fill``: rows the plan does not cover come back as zeros, not uninitialised."""
    _dev(rows_RD, w1_EFD, w3_EFD, w2_EDF)
    _check_experts(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan)
    if gather and plan.row_capacity > 0 and not gather_supported(rows_RD, w1_EFD.shape[1]):
        raise ValueError(
            "the fused token gather needs bf16, D and F multiples of 64 (>= 384), at least one token and a "
            "token matrix below 4 GiB; materialise the rows with permute_rows_fwd instead"
        )
    R = plan.row_capacity if gather else rows_RD.shape[0]
    tok = plan.token_of_row if gather else None
    return _O.grouped_swiglu_fwd(rows_RD, tok, w1_EFD, w3_EFD, w2_EDF, *plan.segments(), R, bool(zero_fill))


def grouped_swiglu_bwd(dy_RD, rows_RD, w1_EFD, w3_EFD, w2_EDF, gate, up, h, plan: PermutePlan,
                       need_drows=True, need_dw=True, gather=False, zero_fill=False):
    _dev(dy_RD, rows_RD)
    if gather and dy_RD.shape[0] > 0 and not gather_supported(rows_RD, w1_EFD.shape[1]):
        raise ValueError("the fused token gather does not cover this dtype / shape")
    tok = plan.token_of_row if gather else None
    drows, dw1, dw3, dw2 = _O.grouped_swiglu_bwd(dy_RD, rows_RD, tok, w1_EFD, w3_EFD, w2_EDF, gate, up, h,
                                                 *plan.segments(), bool(need_drows), bool(need_dw), bool(zero_fill))
    return _opt(drows, need_drows), _opt(dw1, need_dw), _opt(dw3, need_dw), _opt(dw2, need_dw)


def grouped_linear(x_RI, w_EOI, plan: PermutePlan, zero_fill=False):
    """y[r] = x[r] . w[e(r)]^T over the plan's expert segments -- the reference's pluggable
    ``GroupedExperts._grouped_mm(x_TD, weight_EOI, offsets_E)``
    (llmtuner/models/common/moe/experts.py:211-216).  Differentiable in the rows and the weight;
    bf16 with both widths multiples of 64 (>= 384) runs the MFMA kernels, anything else the
    strided fp32-MFMA GEMM.  ``zero_fill``: rows the plan does not cover come back as zeros."""
    _dev(x_RI, w_EOI)
    _dt(x_RI)
    if x_RI.ndim != 2 or w_EOI.ndim != 3 or w_EOI.shape[2] != x_RI.shape[1]:
        raise ValueError(f"grouped weight {tuple(w_EOI.shape)} does not match rows {tuple(x_RI.shape)}")
    if w_EOI.dtype != x_RI.dtype:
        raise TypeError("grouped weight and rows must share one dtype")
    if w_EOI.shape[0] != plan.num_local_experts:
        raise ValueError(f"plan covers {plan.num_local_experts} experts, weights hold {w_EOI.shape[0]}")
    return _O.grouped_linear_fwd(x_RI, w_EOI, *plan.segments(), bool(zero_fill))


def grouped_linear_bwd(dy_RO, x_RI, w_EOI, plan: PermutePlan, need_dx=True, need_dw=True, zero_fill=False):
    """Both gradients of ``grouped_linear``: dx[r] = dy[r] . w[e(r)] and dw[e] = dy[segment e]^T .
    x[segment e] (zeros for an expert without rows).  A gradient that is not asked for is not
    computed and comes back as None."""
    _dev(dy_RO, x_RI, w_EOI)
    dx, dw = _O.grouped_linear_bwd(dy_RO, x_RI, w_EOI, *plan.segments(), bool(need_dx), bool(need_dw), bool(zero_fill))
    return _opt(dx, need_dx), _opt(dw, need_dw)


@torch.compiler.assume_constant_result
def combine_bwd_slots(dtype, D, F):
    """Partials per row of the folded experts+combine backward; 0 when it does not apply.  (A pure
    function of its three constants: a tracing compiler calls it while it traces and keeps the answer.)"""
    if dtype != torch.bfloat16:
        return 0
    return int(_lib.load().mi355_grouped_combine_bwd_slots(_DT[dtype], int(D), int(F)))


def gather_experts_combine(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan: PermutePlan, round_terms=True):
    """out[t] = sum_k weights[t,k] * experts(x)[row(t,k)], with one backward for both halves.

    The forward is the gathered expert product followed by the combine.  The backward never
    forms the expert-major output gradient ``weights * dout`` and never re-reads the expert
    outputs: the dH kernel reads ``dout`` through the plan's token index and scales each row
    in its epilogue, where the same pass yields the gradient of the routing weights (the row's
    unscaled dh times its h, summed over the hidden columns); dW2 contracts the gathered
    ``dout`` rows with ``weights * h``.  Nothing of size (R, D) is kept between forward and
    backward, and of the (R, F) tensors only gate and up -- and when no input asks for a gradient
    (inference) the forward does not write those two either."""
    _dev(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF)
    _check_experts(x_TD, w1_EFD, w3_EFD, w2_EDF, plan)
    if not gather_supported(x_TD, w1_EFD.shape[1]):
        raise ValueError("gather_experts_combine needs bf16 with D and F multiples of 64 (>= 384)")
    differentiable = torch.is_grad_enabled() and any(
        t.requires_grad for t in (x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF))
    out, _gate, _up = _O.gather_experts_combine_fwd(
        x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan.token_of_row, plan.slot_of_row, plan.row_of_slot,
        *plan.segments(), plan.top_k, plan.row_capacity, bool(round_terms), differentiable)
    return out


def rows_experts_combine(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan: PermutePlan, round_terms=True):
    """The same function as ``gather_experts_combine`` for every dtype and shape, in stages: the
    plan's row scatter, the grouped SwiGLU experts, the combine -- as one operator each way (one
    trip through the dispatcher and one autograd node instead of three).  What the module layer
    runs where the folded kernels do not apply (fp32, fp64, widths off the bf16 MFMA path)."""
    _dev(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF)
    _check_experts(x_TD, w1_EFD, w3_EFD, w2_EDF, plan)
    return _O.rows_experts_combine_fwd(
        x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan.row_of_slot, plan.pad_index(), plan.total_rows_1(),
        *plan.segments(), plan.top_k, plan.row_capacity, bool(round_terms))[0]


def combine_row_scale(weights_TK, plan: PermutePlan):
    """row_scale[r] = weights[slot_of_row[r]] (0 for padding rows), fp32."""
    _dev(weights_TK, plan.slot_of_row)
    return _O.combine_row_scale(weights_TK, plan.slot_of_row, plan.row_capacity)


def combine_scores_bwd(dot_partial, plan: PermutePlan):
    _dev(dot_partial)
    return _O.combine_scores_bwd(dot_partial, plan.row_of_slot, plan.num_tokens, plan.top_k)


def grouped_swiglu_combine_bwd(dout_TD, x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, gate, up, plan: PermutePlan,
                               need_dx=True, need_dw=True):
    """Backward of gathered experts + combine in one pass; returns (dx, dw1, dw3, dw2, dweights_TK)."""
    _dev(dout_TD, x_TD)
    if combine_bwd_slots(x_TD.dtype, x_TD.shape[1], w1_EFD.shape[1]) <= 0:
        raise _lib.MI355LibraryError("grouped_swiglu_combine_bwd does not cover this dtype/shape")
    dx, dw1, dw3, dw2, dweights = _O.gather_experts_combine_bwd(
        dout_TD, x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, gate, up, plan.token_of_row, plan.slot_of_row,
        plan.row_of_slot, *plan.segments(), plan.top_k, bool(need_dx), bool(need_dw))
    return _opt(dx, need_dx), _opt(dw1, need_dw), _opt(dw3, need_dw), _opt(dw2, need_dw), dweights


# ====================================================================== profiling hooks
# One MFMA kernel per call on pre-allocated buffers, straight through the C ABI: for
# profilers and per-kernel timing.  Not operators: they write into caller-owned buffers.
STAGES = {"gate_up": 1, "down": 2, "dh": 4, "drows": 8, "dw2": 16, "dw1": 32, "dw3": 64}


def grouped_swiglu_combine_stage(stage: str, buf: dict, plan: PermutePlan):
    """One backward kernel of the folded experts+combine backward on pre-allocated buffers.

    ``buf`` maps dout, rows (the (T, D) tokens), row_scale, w1, w3, w2, gate, up, dgate, dup,
    hs, dot_partial, drows, dw1, dw3, dw2 to device tensors; ``stage`` is one of dh, drows,
    dw2, dw1, dw3.
    """
    x = buf["rows"]
    dev = _dev(x)
    D = x.shape[1]
    R = buf["gate"].shape[0]
    El, F, _ = buf["w1"].shape
    g = lambda k: _p(buf.get(k))
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_grouped_swiglu_combine_bwd(
            g("dout"), g("rows"), _p(plan.token_of_row), x.shape[0], g("row_scale"), g("w1"), g("w3"), g("w2"),
            g("gate"), g("up"), _dt(x), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert),
            _p(plan.tile_row0), _p(plan.num_tiles), plan.tile_capacity, g("dgate"), g("dup"), g("hs"),
            g("dot_partial"), g("drows"), g("dw1"), g("dw3"), g("dw2"), El, D, F, R, STAGES[stage], _stream(dev),
        )
    _lib.check(rc, f"grouped_swiglu_combine_bwd[{stage}]")


def grouped_swiglu_stage(stage: str, buf: dict, plan: PermutePlan):
    """Launch exactly one of the seven bf16 MFMA kernels on pre-allocated buffers.

    ``buf`` maps the C argument names (dy, rows, w1, w3, w2, gate, up, h, y, dgate,
    dup, drows, dw1, dw3, dw2) to device tensors; gate and up may be missing for the gate/up
    stage of a forward-only caller.
    """
    rows = buf["rows"]
    dev = _dev(rows)
    D = rows.shape[1]
    R = buf["h"].shape[0]
    El, F, _ = buf["w1"].shape
    g = lambda k: _p(buf.get(k))
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_grouped_swiglu_stage(
            STAGES[stage], g("dy"), g("rows"), g("token_of_row"), rows.shape[0], g("w1"), g("w3"), g("w2"),
            g("gate"), g("up"), g("h"), g("y"), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert),
            _p(plan.tile_row0), _p(plan.num_tiles), plan.tile_capacity, g("dgate"), g("dup"),
            g("drows"), g("dw1"), g("dw3"), g("dw2"), El, D, F, R, _stream(dev),
        )
    _lib.check(rc, f"grouped_swiglu_stage[{stage}]")


# ====================================================================== differentiable stages
# One name per stage of the block for the module layer (moe/*.py): each is an operator above
# with its autograd formula, so the backward of every stage is the hand-written kernel for it.
#   router_gate              logits = x . W^T in fp32                (custom fwd + bwd GEMMs)
#   route_select             scores -> top-k -> gather -> norm       (fused select, fused VJP)
#   permute_rows             expert-major row gather                 (bwd: K-way row sum)
#   grouped_swiglu           gate/up/SiLU*mul/down grouped GEMMs     (bwd: dX and dW GEMMs)
#   combine                  weighted unpermute                      (bwd: dY and dScore)
#   gather_experts_combine   permute + experts + combine in one node (defined above)


def router_gate(x_TD, weight_ED, logit_bias_E=None):
    """Router projection with fp32 output and fp32 backward GEMMs
    (llmtuner/models/common/linear.py:103-151: ``dX`` comes back in the input dtype and
    ``dW`` in the weight dtype)."""
    return router_gate_fwd(x_TD, weight_ED, logit_bias_E)


def route_select(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                 num_groups=0, num_limited=0, mode=SELECT_TOPK, want_scores=False, want_map=False):
    """Fused score function, expert choice, gather, norm and scale.

    Returns ``(weights_TK, ids_TK, scores_TE or None)`` (plus the bool routing map with
    ``want_map``).  ``scores_TE`` is only materialised (and differentiable) when
    ``want_scores`` is set, which is what an auxiliary loss on the full score map needs."""
    return router_select_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                             num_groups or 0, num_limited or 0, mode, want_scores, want_map)


def route_select_cutoff(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
    """The same selection for a quantile-balanced router in training: also returns the dense
    score map and the (K+1)-th biased score of every token (not differentiable; it only feeds
    the required-bias histogram).  Returns ``(weights_TK, ids_TK, scores_TE, cutoff_T)``."""
    return router_select_cutoff_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale)


def rms_norm(x, weight, epsilon):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last axis; keeps only rstd."""
    return rms_norm_fwd(x, weight, epsilon)[0]


def permute_rows(x_TD, plan):
    """rows[r] = x[token of row r]; backward sums the K row gradients per token."""
    return permute_rows_fwd(x_TD, plan)


def grouped_swiglu(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan, zero_fill=False):
    """y = (silu(rows.w1^T) * rows.w3^T) . w2^T per expert segment."""
    return grouped_swiglu_fwd(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan, zero_fill=zero_fill)[0]


def combine(y_RD, weights_TK, plan, round_terms=True):
    """out[t] = sum_k weights[t,k] * y[row(t,k)]; backward gives dY and dWeights."""
    return combine_fwd(y_RD, weights_TK, plan, round_terms)
