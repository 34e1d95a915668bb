"""Tensor-level wrappers over the C ABI: allocate outputs, pass pointers, check codes.

PyTorch is used here for device memory and the current stream only.  Every function
requires device tensors and raises if given CPU tensors -- the kernels are the only
implementation.
"""

from __future__ import annotations

import os
from dataclasses import dataclass

import torch

from . import _lib

_DT = {torch.float32: 0, torch.bfloat16: 1}
SCORE_FUNCS = {"sigmoid": 0, "softmax": 1, "sqrtsoftplus": 2}
SELECT_TOPK, SELECT_FIXED, SELECT_BALANCED = 0, 1, 2


def _dt(t: torch.Tensor) -> int:
    try:
        return _DT[t.dtype]
    except KeyError:
        raise TypeError(f"MI355 MoE kernels support float32 and bfloat16, got {t.dtype}") from None


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


def _c(t: torch.Tensor) -> torch.Tensor:
    return t if t.is_contiguous() else t.contiguous()


def tile_m(dtype: torch.dtype = torch.bfloat16) -> int:
    return int(_lib.load().mi355_grouped_tile_m(_DT[dtype]))


# ------------------------------------------------------------------ router
def router_gate_fwd(x_TD, w_ED, logit_bias_E=None):
    dev = _dev(x_TD, w_ED, logit_bias_E)
    x_TD, w_ED = _c(x_TD), _c(w_ED)
    T, D = x_TD.shape
    E = w_ED.shape[0]
    if w_ED.shape[1] != D:
        raise ValueError(f"gate weight {tuple(w_ED.shape)} does not match input dim {D}")
    bias = None if logit_bias_E is None else _c(logit_bias_E.float())
    out = torch.empty(T, E, dtype=torch.float32, device=dev)
    lib = _lib.load()
    nbytes = lib.mi355_router_gate_fwd_workspace_bytes(T, D, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    with torch.cuda.device(dev):
        rc = lib.mi355_router_gate_fwd(
            _p(x_TD), _dt(x_TD), _p(w_ED), _dt(w_ED), _p(bias), _p(out), _p(ws), T, D, E, _stream(dev)
        )
    _lib.check(rc, "router_gate_fwd")
    return out


def router_gate_bwd(dlogits_TE, x_TD, w_ED, need_dx=True, need_dw=True):
    dev = _dev(dlogits_TE, x_TD, w_ED)
    dlogits_TE, x_TD, w_ED = _c(dlogits_TE.float()), _c(x_TD), _c(w_ED)
    T, D = x_TD.shape
    E = w_ED.shape[0]
    lib = _lib.load()
    dx = torch.empty_like(x_TD) if need_dx else None
    dw = torch.empty_like(w_ED) if need_dw else None
    nbytes = lib.mi355_router_gate_bwd_workspace_bytes(T, D, E)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=dev) if nbytes else None
    with torch.cuda.device(dev):
        rc = lib.mi355_router_gate_bwd(
            _p(dlogits_TE), _p(x_TD), _dt(x_TD), _p(w_ED), _dt(w_ED), _p(dx), _p(dw), _p(ws),
            T, D, E, _stream(dev),
        )
    _lib.check(rc, "router_gate_bwd")
    return dx, dw


def router_select_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                      num_groups=0, num_limited=0, mode=SELECT_TOPK, want_scores=False):
    dev = _dev(logits_TE, expert_bias_E)
    if logits_TE.dtype != torch.float32:
        raise TypeError("router logits must be float32")
    logits_TE = _c(logits_TE)
    T, E = logits_TE.shape
    bias = None if expert_bias_E is None else _c(expert_bias_E.float())
    weights = torch.empty(T, top_k, dtype=torch.float32, device=dev)
    ids = torch.empty(T, top_k, dtype=torch.int64, device=dev)
    scores = torch.empty(T, E, dtype=torch.float32, device=dev) if want_scores else None
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_router_select_fwd(
            _p(logits_TE), _p(bias), _p(weights), _p(ids), _p(scores), T, E, top_k,
            SCORE_FUNCS[score_func], int(route_norm), float(route_scale), int(num_groups or 0),
            int(num_limited or 0), mode, _stream(dev),
        )
    _lib.check(rc, "router_select_fwd")
    return weights, ids, scores


def router_select_cutoff_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
    """Biased top-k plus the (K+1)-th biased score of every token: returns
    ``(weights_TK, ids_TK, scores_TE, cutoff_T)``."""
    dev = _dev(logits_TE, expert_bias_E)
    if logits_TE.dtype != torch.float32:
        raise TypeError("router logits must be float32")
    logits_TE = _c(logits_TE)
    T, E = logits_TE.shape
    bias = None if expert_bias_E is None else _c(expert_bias_E.float())
    weights = torch.empty(T, top_k, dtype=torch.float32, device=dev)
    ids = torch.empty(T, top_k, dtype=torch.int64, device=dev)
    scores = torch.empty(T, E, dtype=torch.float32, device=dev)
    cutoff = torch.empty(T, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_router_select_cutoff_fwd(
            _p(logits_TE), _p(bias), _p(weights), _p(ids), _p(scores), _p(cutoff), T, E, top_k,
            SCORE_FUNCS[score_func], int(route_norm), float(route_scale), _stream(dev),
        )
    _lib.check(rc, "router_select_cutoff_fwd")
    return weights, ids, scores, cutoff


def quantile_observe(histogram_EB, scores_TE, cutoff_T, expert_bias_E, padding_mask_T=None):
    """Accumulates the required-bias histogram in place (int64 ``(E, B)``)."""
    dev = _dev(histogram_EB, scores_TE, cutoff_T, expert_bias_E, padding_mask_T)
    if histogram_EB.dtype != torch.int64 or not histogram_EB.is_contiguous():
        raise TypeError("histogram_EB must be a contiguous int64 tensor")
    scores_TE = _c(scores_TE.float())
    T, E = scores_TE.shape
    if histogram_EB.shape[0] != E or cutoff_T.numel() != T or expert_bias_E.numel() != E:
        raise ValueError(
            f"quantile_observe: histogram {tuple(histogram_EB.shape)}, scores {(T, E)}, "
            f"cutoff {tuple(cutoff_T.shape)} and bias {tuple(expert_bias_E.shape)} do not agree"
        )
    cutoff_T = _c(cutoff_T.float().reshape(-1))
    bias = _c(expert_bias_E.float())
    pad = None
    if padding_mask_T is not None:
        if padding_mask_T.dtype != torch.bool or padding_mask_T.numel() != T:
            raise ValueError("padding_mask_T must be a bool tensor with one entry per token")
        pad = _c(padding_mask_T.reshape(-1)).view(torch.uint8)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_quantile_observe(
            _p(scores_TE), _p(cutoff_T), _p(bias), _p(pad), _p(histogram_EB), T, E,
            histogram_EB.shape[1], _stream(dev),
        )
    _lib.check(rc, "quantile_observe")


def quantile_estimate(histogram_EB, expert_bias_E, top_k):
    """The next mean-centred expert bias (new tensor, dtype of ``expert_bias_E``)."""
    dev = _dev(histogram_EB, expert_bias_E)
    if histogram_EB.dtype != torch.int64:
        raise TypeError("histogram_EB must be int64")
    histogram_EB = _c(histogram_EB)
    E, B = histogram_EB.shape
    bias = _c(expert_bias_E.float())
    out = torch.empty(E, dtype=torch.float32, device=dev)
    ws = torch.empty(2 * E, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_quantile_estimate(
            _p(histogram_EB), _p(bias), _p(out), _p(ws), E, top_k, B, _stream(dev)
        )
    _lib.check(rc, "quantile_estimate")
    return out.to(expert_bias_E.dtype)


def rms_norm_fwd(x, weight, epsilon):
    """Returns ``(y, rstd)``; ``x`` is ``(..., D)``, ``weight`` ``(D,)`` of the same dtype."""
    dev = _dev(x, weight)
    if x.dtype != weight.dtype:
        raise TypeError(f"rms_norm: input ({x.dtype}) and weight ({weight.dtype}) must share a dtype")
    x, weight = _c(x), _c(weight)
    D = weight.numel()
    rows = x.numel() // D
    y = torch.empty_like(x)
    rstd = torch.empty(rows, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_rms_norm_fwd(_p(x), _p(weight), _dt(x), _p(y), _p(rstd), rows, D,
                                            float(epsilon), _stream(dev))
    _lib.check(rc, "rms_norm_fwd")
    return y, rstd


def rms_norm_bwd(dy, x, weight, rstd, need_dx=True, need_dw=True):
    """Returns ``(dx or None, dweight or None)``."""
    dev = _dev(dy, x, weight, rstd)
    dy, x, weight = _c(dy), _c(x), _c(weight)
    if dy.dtype != x.dtype:
        dy = dy.to(x.dtype)
    D = weight.numel()
    rows = x.numel() // D
    lib = _lib.load()
    dx = torch.empty_like(x) if need_dx else None
    dw = torch.empty_like(weight) if need_dw else None
    ws = torch.empty(max(lib.mi355_rms_norm_bwd_workspace_bytes(rows, D), 4), dtype=torch.uint8,
                     device=dev) if need_dw else None
    with torch.cuda.device(dev):
        rc = lib.mi355_rms_norm_bwd(_p(dy), _p(x), _p(weight), _p(rstd), _dt(x), _p(dx), _p(dw), _p(ws),
                                    rows, D, _stream(dev))
    _lib.check(rc, "rms_norm_bwd")
    return dx, dw


def router_select_bwd(logits_TE, ids_TK, dweights_TK, dscores_TE, score_func, route_norm,
                      route_scale, mode=SELECT_TOPK):
    dev = _dev(logits_TE, ids_TK, dweights_TK, dscores_TE)
    logits_TE, ids_TK = _c(logits_TE), _c(ids_TK)
    T, E = logits_TE.shape
    K = ids_TK.shape[1]
    dweights_TK = None if dweights_TK is None else _c(dweights_TK.float())
    dscores_TE = None if dscores_TE is None else _c(dscores_TE.float())
    out = torch.empty_like(logits_TE)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_router_select_bwd(
            _p(logits_TE), _p(ids_TK), _p(dweights_TK), _p(dscores_TE), _p(out), T, E, K,
            SCORE_FUNCS[score_func], int(route_norm), float(route_scale), mode, _stream(dev),
        )
    _lib.check(rc, "router_select_bwd")
    return out


def balance_loss_fwd(scores_TE, routing_map_TE, padding_mask_T=None):
    """Returns (loss 0-d fp32, f_E) of the per-forward load-balance loss."""
    dev = _dev(scores_TE, routing_map_TE, padding_mask_T)
    if scores_TE.dtype != torch.float32:
        raise TypeError("router scores must be float32")
    scores_TE = _c(scores_TE)
    T, E = scores_TE.shape
    if routing_map_TE.shape != scores_TE.shape:
        raise ValueError(f"routing map {tuple(routing_map_TE.shape)} does not match scores {tuple(scores_TE.shape)}")
    as_bytes = lambda m: _c(m).view(torch.uint8) if m.dtype == torch.bool else _c(m.ne(0)).view(torch.uint8)
    rmap = as_bytes(routing_map_TE)
    pad = None if padding_mask_T is None else as_bytes(padding_mask_T)
    lib = _lib.load()
    out = torch.empty(1 + E, dtype=torch.float32, device=dev)
    ws = torch.empty(max(lib.mi355_balance_loss_workspace_bytes(T, E), 4), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.mi355_balance_loss_fwd(_p(scores_TE), _p(rmap), _p(pad), _p(out), out[1:].data_ptr(), _p(ws),
                                        T, E, _stream(dev))
    _lib.check(rc, "balance_loss_fwd")
    return out[0], out[1:]


def balance_loss_bwd(scores_TE, f_E, grad_loss, padding_mask_T=None):
    dev = _dev(scores_TE, f_E, grad_loss, padding_mask_T)
    scores_TE = _c(scores_TE)
    T, E = scores_TE.shape
    pad = None if padding_mask_T is None else _c(padding_mask_T).view(torch.uint8)
    g = _c(grad_loss.float().reshape(1))
    out = torch.empty_like(scores_TE)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_balance_loss_bwd(_p(scores_TE), _p(_c(f_E)), _p(pad), _p(g), _p(out), T, E,
                                                _stream(dev))
    _lib.check(rc, "balance_loss_bwd")
    return out


# ------------------------------------------------------------------ plan
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


def permute_plan(ids_TK, num_experts, local_lo=0, local_hi=None, align=1) -> PermutePlan:
    dev = _dev(ids_TK)
    if ids_TK.dtype != torch.int64:
        ids_TK = ids_TK.to(torch.int64)
    ids_TK = _c(ids_TK)
    T, K = ids_TK.shape
    E = int(num_experts)
    hi = E if local_hi is None else int(local_hi)
    lo = int(local_lo)
    El = hi - lo
    N = T * K
    tm = tile_m()
    row_cap = N + (El * (align - 1) if align > 1 else 0)
    tile_cap = N // tm + El + 1
    lib = _lib.load()
    i32 = dict(dtype=torch.int32, device=dev)
    # one allocation for the small arrays, one for the per-slot / per-row ones
    small = torch.empty(E + (El + 1) + 2 * El + 2 * tile_cap + 1, **i32)
    o = 0
    counts_E = small[o:o + E]; o += E
    seg_offsets = small[o:o + El + 1]; o += El + 1
    # the library writes 2*El ints here: the counts, then the experts by descending count
    seg_counts = small[o:o + El]; expert_order = small[o + El:o + 2 * El]; o += 2 * El
    tile_expert = small[o:o + tile_cap]; o += tile_cap
    tile_row0 = small[o:o + tile_cap]; o += tile_cap
    num_tiles = small[o:o + 1]
    row_of_slot = torch.empty(N, **i32)
    rows2 = torch.empty(2, row_cap, **i32)
    slot_of_row, token_of_row = rows2[0], rows2[1]
    ws = torch.empty(lib.mi355_permute_plan_workspace_bytes(T, K, E), dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.mi355_permute_plan(
            _p(ids_TK), T, K, E, lo, hi, align, tm, _p(counts_E), _p(seg_offsets), _p(seg_counts),
            _p(row_of_slot), _p(slot_of_row), _p(token_of_row), row_cap, _p(tile_expert), _p(tile_row0),
            _p(num_tiles), tile_cap, _p(ws), _stream(dev),
        )
    _lib.check(rc, "permute_plan")
    return PermutePlan(T, K, E, lo, hi, align, tm, row_cap, tile_cap, counts_E, seg_offsets,
                       seg_counts, row_of_slot, slot_of_row, token_of_row, tile_expert, tile_row0, num_tiles,
                       expert_order)


def segments_from_counts(counts_e, total_rows: int) -> PermutePlan:
    """Plan for rows that are already expert-major with ``counts_e`` rows each."""
    dev = _dev(counts_e)
    counts = _c(counts_e.to(torch.int32))
    El = counts.shape[0]
    tm = tile_m()
    tile_cap = total_rows // tm + El + 1
    i32 = dict(dtype=torch.int32, device=dev)
    small = torch.empty((El + 1) + 2 * El + 2 * tile_cap + 1, **i32)
    o = 0
    seg_offsets = small[o:o + El + 1]; o += El + 1
    seg_counts = small[o:o + El]; expert_order = small[o + El:o + 2 * El]; o += 2 * El
    tile_expert = small[o:o + tile_cap]; o += tile_cap
    tile_row0 = small[o:o + tile_cap]; o += tile_cap
    num_tiles = small[o:o + 1]
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_segments_from_counts(
            _p(counts), El, tm, total_rows, _p(seg_offsets), _p(seg_counts), _p(tile_expert), _p(tile_row0),
            _p(num_tiles), tile_cap, _stream(dev),
        )
    _lib.check(rc, "segments_from_counts")
    return PermutePlan(0, 1, El, 0, El, 1, tm, total_rows, tile_cap, None, seg_offsets, seg_counts,
                       None, None, None, tile_expert, tile_row0, num_tiles, expert_order)


# ------------------------------------------------------------------ row movers
def permute_rows_fwd(x_TD, plan: PermutePlan):
    dev = _dev(x_TD, plan.slot_of_row)
    x_TD = _c(x_TD)
    T, D = x_TD.shape
    rows = torch.empty(plan.row_capacity, D, dtype=x_TD.dtype, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_permute_rows_fwd(
            _p(x_TD), _dt(x_TD), _p(plan.slot_of_row), _p(plan.total_rows), _p(rows), T, D,
            plan.top_k, plan.row_capacity, _stream(dev),
        )
    _lib.check(rc, "permute_rows_fwd")
    return rows


def permute_rows_bwd(drows_RD, plan: PermutePlan):
    dev = _dev(drows_RD, plan.row_of_slot)
    drows_RD = _c(drows_RD)
    D = drows_RD.shape[1]
    dx = torch.empty(plan.num_tokens, D, dtype=drows_RD.dtype, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_permute_rows_bwd(
            _p(drows_RD), _dt(drows_RD), _p(plan.row_of_slot), _p(dx), plan.num_tokens, D,
            plan.top_k, _stream(dev),
        )
    _lib.check(rc, "permute_rows_bwd")
    return dx


def combine_fwd(y_RD, weights_TK, plan: PermutePlan, round_terms=True, out_dtype=None):
    dev = _dev(y_RD, weights_TK, plan.row_of_slot)
    y_RD, weights_TK = _c(y_RD), _c(weights_TK.float())
    D = y_RD.shape[1]
    out = torch.empty(plan.num_tokens, D, dtype=y_RD.dtype, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_combine_fwd(
            _p(y_RD), _dt(y_RD), _p(weights_TK), _p(plan.row_of_slot), _p(out), plan.num_tokens, D,
            plan.top_k, int(round_terms), _stream(dev),
        )
    _lib.check(rc, "combine_fwd")
    return out


def combine_bwd(dout_TD, y_RD, weights_TK, plan: PermutePlan, zero_padding=True):
    dev = _dev(dout_TD, y_RD, weights_TK)
    dout_TD, y_RD, weights_TK = _c(dout_TD), _c(y_RD), _c(weights_TK.float())
    if dout_TD.dtype != y_RD.dtype:
        dout_TD = dout_TD.to(y_RD.dtype)
    D = y_RD.shape[1]
    dy = torch.empty_like(y_RD)
    dw = torch.empty(plan.num_tokens, plan.top_k, dtype=torch.float32, device=dev)
    pad = plan.slot_of_row if (zero_padding and plan.align > 1) else None
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_combine_bwd(
            _p(dout_TD), _p(y_RD), _dt(y_RD), _p(weights_TK), _p(plan.row_of_slot), _p(pad),
            _p(plan.total_rows), _p(dy), _p(dw), plan.num_tokens, D, plan.top_k,
            y_RD.shape[0], _stream(dev),
        )
    _lib.check(rc, "combine_bwd")
    return dy, dw


# ------------------------------------------------------------------ experts
def gather_supported(x_TD, hidden_dim: int) -> bool:
    """The fused token gather exists for the bf16 MFMA kernels (D, F multiples of 64, at
    least 384: the library's own condition for that path)."""
    D = x_TD.shape[-1]
    return (x_TD.dtype == torch.bfloat16 and D % 64 == 0 and hidden_dim % 64 == 0
            and D >= 384 and hidden_dim >= 384 and x_TD.shape[0] * D < 2**31)


def grouped_swiglu_fwd(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan: PermutePlan, gather=False):
    """``gather=True``: ``rows_RD`` is the (T, D) token matrix, read through ``plan.token_of_row``."""
    dev = _dev(rows_RD, w1_EFD, w3_EFD, w2_EDF)
    rows_RD, w1_EFD, w3_EFD, w2_EDF = _c(rows_RD), _c(w1_EFD), _c(w3_EFD), _c(w2_EDF)
    D = rows_RD.shape[1]
    R = plan.row_capacity if gather else rows_RD.shape[0]
    tok = plan.token_of_row if gather else None
    El, F, D2 = w1_EFD.shape
    if D2 != D or w3_EFD.shape != w1_EFD.shape or w2_EDF.shape != (El, D, F):
        raise ValueError("expert weight shapes do not match (E,F,D)/(E,F,D)/(E,D,F)")
    if not (w1_EFD.dtype == w3_EFD.dtype == w2_EDF.dtype == rows_RD.dtype):
        raise TypeError("expert weights and rows must share one dtype")
    if El != plan.num_local_experts:
        raise ValueError(f"plan covers {plan.num_local_experts} experts, weights hold {El}")
    mk = lambda n: torch.empty(R, n, dtype=rows_RD.dtype, device=dev)
    gate, up, h, y = mk(F), mk(F), mk(F), mk(D)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_grouped_swiglu_fwd(
            _p(rows_RD), _p(tok), _p(w1_EFD), _p(w3_EFD), _p(w2_EDF), _dt(rows_RD),
            _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert), _p(plan.tile_row0),
            _p(plan.num_tiles), plan.tile_capacity, _p(gate), _p(up), _p(h), _p(y), El, D, F, R,
            _stream(dev),
        )
    _lib.check(rc, "grouped_swiglu_fwd")
    return y, gate, up, h


def grouped_swiglu_bwd(dy_RD, rows_RD, w1_EFD, w3_EFD, w2_EDF, gate, up, h, plan: PermutePlan,
                       need_drows=True, need_dw=True, gather=False):
    dev = _dev(dy_RD, rows_RD)
    dy_RD = _c(dy_RD)
    w1_EFD, w3_EFD, w2_EDF = _c(w1_EFD), _c(w3_EFD), _c(w2_EDF)
    D = rows_RD.shape[1]
    R = dy_RD.shape[0]
    tok = plan.token_of_row if gather else None
    El, F, _ = w1_EFD.shape
    dgate, dup = torch.empty_like(gate), torch.empty_like(up)
    drows = torch.empty(R, D, dtype=rows_RD.dtype, device=dev) if need_drows else None
    dw1 = torch.empty_like(w1_EFD) if need_dw else None
    dw3 = torch.empty_like(w3_EFD) if need_dw else None
    dw2 = torch.empty_like(w2_EDF) if need_dw else None
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_grouped_swiglu_bwd(
            _p(dy_RD), _p(rows_RD), _p(tok), _p(w1_EFD), _p(w3_EFD), _p(w2_EDF), _p(gate), _p(up),
            _p(h), _dt(rows_RD), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert),
            _p(plan.tile_row0), _p(plan.num_tiles), plan.tile_capacity, _p(dgate), _p(dup),
            _p(drows), _p(dw1), _p(dw3), _p(dw2), El, D, F, R, _stream(dev),
        )
    _lib.check(rc, "grouped_swiglu_bwd")
    return drows, dw1, dw3, dw2


# False sends RoutedExperts through the two-call backward (combine, then experts) also where
# the folded one applies (MI355_FOLD_COMBINE=0 in the environment does the same).
FOLD_COMBINE = os.environ.get("MI355_FOLD_COMBINE", "1") != "0"


def combine_bwd_slots(dtype, D, F):
    """Partials per row of the folded experts+combine backward; 0 when it does not apply."""
    if dtype != torch.bfloat16 or not FOLD_COMBINE:
        return 0
    return int(_lib.load().mi355_grouped_combine_bwd_slots(_DT[dtype], int(D), int(F)))


def combine_row_scale(weights_TK, plan: PermutePlan):
    """row_scale[r] = weights[slot_of_row[r]] (0 for padding rows), fp32."""
    dev = _dev(weights_TK, plan.slot_of_row)
    weights_TK = _c(weights_TK.float())
    R = plan.row_capacity
    out = torch.empty(R, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_combine_row_scale(
            _p(weights_TK), _p(plan.slot_of_row), _p(out), plan.num_tokens, plan.top_k, R, _stream(dev),
        )
    _lib.check(rc, "combine_row_scale")
    return out


def grouped_swiglu_combine_bwd(dout_TD, x_TD, row_scale_R, w1_EFD, w3_EFD, w2_EDF, gate, up, plan: PermutePlan,
                               need_drows=True, need_dw=True, sum_rows=False):
    """Backward of gathered experts + combine in one pass; returns (drows, dw1, dw3, dw2, dweights_TK).

    ``sum_rows``: return ``dx`` (T, D), the K-way row sum of ``drows``, in its place.  The sum
    then runs right behind the kernel that wrote ``drows``, while those rows are still in the
    memory-side cache, and the weight-gradient kernels follow; summed after them it finds its
    input gone to HBM.
    """
    dev = _dev(dout_TD, x_TD)
    dout_TD, x_TD = _c(dout_TD), _c(x_TD)
    if dout_TD.dtype != x_TD.dtype:
        dout_TD = dout_TD.to(x_TD.dtype)
    w1_EFD, w3_EFD, w2_EDF = _c(w1_EFD), _c(w3_EFD), _c(w2_EDF)
    D = x_TD.shape[1]
    R = gate.shape[0]
    El, F, _ = w1_EFD.shape
    lib = _lib.load()
    slots = combine_bwd_slots(x_TD.dtype, D, F)
    if slots <= 0:
        raise _lib.MI355LibraryError("grouped_swiglu_combine_bwd does not cover this dtype/shape/layout")
    dgate, dup, hs = torch.empty_like(gate), torch.empty_like(up), torch.empty_like(gate)
    partial = torch.empty(R, slots, dtype=torch.float32, device=dev)
    drows = torch.empty(R, D, dtype=x_TD.dtype, device=dev) if need_drows else None
    dw1 = torch.empty_like(w1_EFD) if need_dw else None
    dw3 = torch.empty_like(w3_EFD) if need_dw else None
    dw2 = torch.empty_like(w2_EDF) if need_dw else None
    def run(stages):
        with torch.cuda.device(dev):
            rc = lib.mi355_grouped_swiglu_combine_bwd(
                _p(dout_TD), _p(x_TD), _p(plan.token_of_row), _p(row_scale_R), _p(w1_EFD), _p(w3_EFD), _p(w2_EDF),
                _p(gate), _p(up), _dt(x_TD), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert),
                _p(plan.tile_row0), _p(plan.num_tiles), plan.tile_capacity, _p(dgate), _p(dup), _p(hs), _p(partial),
                _p(drows), _p(dw1), _p(dw3), _p(dw2), El, D, F, R, stages, _stream(dev),
            )
        _lib.check(rc, "grouped_swiglu_combine_bwd")

    if not (sum_rows and need_drows and need_dw and R > 0):
        run(0)
        if sum_rows and drows is not None:
            drows = permute_rows_bwd(drows, plan)
        return drows, dw1, dw3, dw2, combine_scores_bwd(partial, plan)
    run(STAGES["dh"] | STAGES["drows"])
    dx = permute_rows_bwd(drows, plan)
    dweights = combine_scores_bwd(partial, plan)
    run(STAGES["dw2"] | STAGES["dw1"] | STAGES["dw3"])
    return dx, dw1, dw3, dw2, dweights


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
            g("dout"), g("rows"), _p(plan.token_of_row), g("row_scale"), g("w1"), g("w3"), g("w2"), g("gate"),
            g("up"), _dt(x), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert), _p(plan.tile_row0),
            _p(plan.num_tiles), plan.tile_capacity, g("dgate"), g("dup"), g("hs"), g("dot_partial"), g("drows"),
            g("dw1"), g("dw3"), g("dw2"), El, D, F, R, STAGES[stage], _stream(dev),
        )
    _lib.check(rc, f"grouped_swiglu_combine_bwd[{stage}]")


def combine_scores_bwd(dot_partial, plan: PermutePlan):
    dev = _dev(dot_partial)
    dweights = torch.empty(plan.num_tokens, plan.top_k, dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_combine_scores_bwd(
            _p(dot_partial), dot_partial.shape[1], _p(plan.row_of_slot), _p(dweights), plan.num_tokens, plan.top_k,
            dot_partial.shape[0], _stream(dev),
        )
    _lib.check(rc, "combine_scores_bwd")
    return dweights


def grouped_swiglu_stage(stage: str, buf: dict, plan: PermutePlan):
    """Launch exactly one of the seven bf16 MFMA kernels on pre-allocated buffers.

    ``buf`` maps the C argument names (dy, rows, w1, w3, w2, gate, up, h, y, dgate,
    dup, drows, dw1, dw3, dw2) to device tensors.
    """
    rows = buf["rows"]
    dev = _dev(rows)
    D = rows.shape[1]
    R = buf["gate"].shape[0]
    El, F, _ = buf["w1"].shape
    g = lambda k: _p(buf.get(k))
    with torch.cuda.device(dev):
        rc = _lib.load().mi355_grouped_swiglu_stage(
            STAGES[stage], g("dy"), g("rows"), g("token_of_row"), g("w1"), g("w3"), g("w2"), g("gate"), g("up"), g("h"),
            g("y"), _p(plan.seg_offsets), _p(plan.seg_counts), _p(plan.tile_expert),
            _p(plan.tile_row0), _p(plan.num_tiles), plan.tile_capacity, g("dgate"), g("dup"),
            g("drows"), g("dw1"), g("dw3"), g("dw2"), El, D, F, R, _stream(dev),
        )
    _lib.check(rc, f"grouped_swiglu_stage[{stage}]")
