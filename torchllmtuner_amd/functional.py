"""Autograd nodes over the HIP kernels, one per stage of the MoE block.

Each node's backward is the hand-written kernel for that stage; nothing here falls
back to PyTorch math.  Stages (reference lines each replaces are cited in
include/mi355_moe.h):

  router_gate     logits = x . W^T in fp32                (custom fwd + bwd GEMMs)
  route_select    scores -> top-k -> gather -> norm       (fused select, fused VJP)
  permute_rows    expert-major row gather                 (bwd: K-way row sum)
  grouped_swiglu  gate/up/SiLU*mul/down grouped GEMMs     (bwd: dX and dW GEMMs)
                  (gather_grouped_swiglu fuses permute_rows into the GEMM operand loads)
  combine         weighted unpermute                      (bwd: dY and dScore)
"""

from __future__ import annotations

import torch
from torch.autograd.function import once_differentiable

from . import ops


class RouterGateLinearFunction(torch.autograd.Function):
    """Router projection with fp32 output and fp32 backward GEMMs.

    Mirrors llmtuner/models/common/linear.py:103-151: ``dX`` comes back in the
    input dtype and ``dW`` in the weight dtype.
    """

    @staticmethod
    def forward(ctx, input_TD, weight_ED, logit_bias_E=None):
        ctx.save_for_backward(input_TD, weight_ED)
        ctx.has_bias = logit_bias_E is not None
        ctx.bias_dtype = None if logit_bias_E is None else logit_bias_E.dtype
        return ops.router_gate_fwd(input_TD, weight_ED, logit_bias_E)

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_TE):
        x, w = ctx.saved_tensors
        dx, dw = ops.router_gate_bwd(
            grad_TE, x, w, need_dx=ctx.needs_input_grad[0], need_dw=ctx.needs_input_grad[1]
        )
        db = None
        if ctx.has_bias and ctx.needs_input_grad[2]:
            db = grad_TE.float().sum(dim=0).to(ctx.bias_dtype)
        return dx, dw, db


class RouteSelectFunction(torch.autograd.Function):
    """Fused score function, expert choice, gather, norm and scale.

    Returns ``(weights_TK, ids_TK, scores_TE or None)``.  ``scores_TE`` is only
    materialised (and differentiable) when ``want_scores`` is set, which is what an
    auxiliary loss on the full score map needs.
    """

    @staticmethod
    def forward(ctx, logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                num_groups, num_limited, mode, want_scores):
        weights, ids, scores = ops.router_select_fwd(
            logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
            num_groups, num_limited, mode, want_scores,
        )
        ctx.save_for_backward(logits_TE, ids)
        ctx.cfg = (score_func, route_norm, route_scale, mode)
        ctx.mark_non_differentiable(ids)
        if scores is None:
            return weights, ids, None
        return weights, ids, scores

    @staticmethod
    @once_differentiable
    def backward(ctx, dweights, _dids, dscores):
        logits, ids = ctx.saved_tensors
        score_func, route_norm, route_scale, mode = ctx.cfg
        dlogits = None
        if ctx.needs_input_grad[0]:
            dlogits = ops.router_select_bwd(
                logits, ids, dweights, dscores, score_func, route_norm, route_scale, mode
            )
        return (dlogits,) + (None,) * 9


class RouteSelectCutoffFunction(torch.autograd.Function):
    """The same selection for a quantile-balanced router in training: also returns the
    dense score map and the (K+1)-th biased score of every token (not differentiable;
    it only feeds the required-bias histogram).

    Returns ``(weights_TK, ids_TK, scores_TE, cutoff_T)``.
    """

    @staticmethod
    def forward(ctx, logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
        weights, ids, scores, cutoff = ops.router_select_cutoff_fwd(
            logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale
        )
        ctx.save_for_backward(logits_TE, ids)
        ctx.cfg = (score_func, route_norm, route_scale)
        ctx.set_materialize_grads(False)  # no dense zero gradient for an unused score map
        ctx.mark_non_differentiable(ids, cutoff)
        return weights, ids, scores, cutoff

    @staticmethod
    @once_differentiable
    def backward(ctx, dweights, _dids, dscores, _dcutoff):
        logits, ids = ctx.saved_tensors
        score_func, route_norm, route_scale = ctx.cfg
        dlogits = None
        if ctx.needs_input_grad[0]:
            dlogits = ops.router_select_bwd(
                logits, ids, dweights, dscores, score_func, route_norm, route_scale, ops.SELECT_TOPK
            )
        return (dlogits,) + (None,) * 5


class RMSNormFunction(torch.autograd.Function):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last axis; keeps only rstd."""

    @staticmethod
    def forward(ctx, x, weight, epsilon):
        y, rstd = ops.rms_norm_fwd(x, weight, epsilon)
        ctx.save_for_backward(x, weight, rstd)
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy):
        x, weight, rstd = ctx.saved_tensors
        dx, dw = ops.rms_norm_bwd(dy, x, weight, rstd, ctx.needs_input_grad[0], ctx.needs_input_grad[1])
        return dx, dw, None


class PermuteRowsFunction(torch.autograd.Function):
    """rows[r] = x[token of row r]; backward sums the K row gradients per token."""

    @staticmethod
    def forward(ctx, x_TD, plan):
        ctx.plan = plan
        return ops.permute_rows_fwd(x_TD, plan)

    @staticmethod
    @once_differentiable
    def backward(ctx, drows):
        return ops.permute_rows_bwd(drows, ctx.plan), None


class GroupedSwiGLUFunction(torch.autograd.Function):
    """y = (silu(rows.w1^T) * rows.w3^T) . w2^T per expert segment."""

    @staticmethod
    def forward(ctx, rows_RD, w1_EFD, w3_EFD, w2_EDF, plan):
        y, gate, up, h = ops.grouped_swiglu_fwd(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan)
        ctx.save_for_backward(rows_RD, w1_EFD, w3_EFD, w2_EDF, gate, up, h)
        ctx.plan = plan
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy):
        rows, w1, w3, w2, gate, up, h = ctx.saved_tensors
        need_dw = any(ctx.needs_input_grad[1:4])
        drows, dw1, dw3, dw2 = ops.grouped_swiglu_bwd(
            dy, rows, w1, w3, w2, gate, up, h, ctx.plan,
            need_drows=ctx.needs_input_grad[0], need_dw=need_dw,
        )
        return drows, dw1, dw3, dw2, None


class GatherGroupedSwiGLUFunction(torch.autograd.Function):
    """Token gather fused into the expert GEMMs: y rows from the unpermuted (T, D) tokens.

    Forward never materialises the expert-major copy of the tokens: the gate/up kernel
    reads ``x[token_of_row[r]]`` directly, and nothing of size (R, D) is kept for the
    backward.  The weight-gradient kernels read their K rows through the same index (the
    row numbers of a K step are fetched one step ahead of its data), and ``dx`` is the
    K-way row sum of the expert-major input gradient.
    """

    @staticmethod
    def forward(ctx, x_TD, w1_EFD, w3_EFD, w2_EDF, plan):
        y, gate, up, h = ops.grouped_swiglu_fwd(x_TD, w1_EFD, w3_EFD, w2_EDF, plan, gather=True)
        ctx.save_for_backward(x_TD, w1_EFD, w3_EFD, w2_EDF, gate, up, h)
        ctx.plan = plan
        return y

    @staticmethod
    @once_differentiable
    def backward(ctx, dy):
        x, w1, w3, w2, gate, up, h = ctx.saved_tensors
        drows, dw1, dw3, dw2 = ops.grouped_swiglu_bwd(
            dy, x, w1, w3, w2, gate, up, h, ctx.plan,
            need_drows=ctx.needs_input_grad[0], need_dw=any(ctx.needs_input_grad[1:4]), gather=True,
        )
        dx = ops.permute_rows_bwd(drows, ctx.plan) if drows is not None else None
        return dx, dw1, dw3, dw2, None


class GatherExpertsCombineFunction(torch.autograd.Function):
    """out[t] = sum_k weights[t,k] * experts(x)[row(t,k)] with one backward for both halves.

    The forward is the gathered expert product followed by the combine.  The backward never
    forms the expert-major output gradient ``weights * dout`` and never re-reads the expert
    outputs: the dH kernel reads ``dout`` through the plan's token index and scales each row
    in its epilogue, where the same pass yields the gradient of the routing weights (the row's
    unscaled dh times its h, summed over the hidden columns); dW2 contracts the gathered
    ``dout`` rows with ``weights * h``.  Nothing of size (R, D) is kept between forward and
    backward, and of the (R, F) tensors only gate and up.
    """

    @staticmethod
    def forward(ctx, x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan, round_terms):
        y, gate, up, _h = ops.grouped_swiglu_fwd(x_TD, w1_EFD, w3_EFD, w2_EDF, plan, gather=True)
        out = ops.combine_fwd(y, weights_TK, plan, round_terms)
        ctx.save_for_backward(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, gate, up)
        ctx.plan = plan
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, dout):
        x, weights, w1, w3, w2, gate, up = ctx.saved_tensors
        row_scale = ops.combine_row_scale(weights, ctx.plan)
        dx, dw1, dw3, dw2, dweights = ops.grouped_swiglu_combine_bwd(
            dout, x, row_scale, w1, w3, w2, gate, up, ctx.plan,
            need_drows=ctx.needs_input_grad[0], need_dw=any(ctx.needs_input_grad[2:5]), sum_rows=True,
        )
        return dx, dweights.to(weights.dtype), dw1, dw3, dw2, None, None


class CombineFunction(torch.autograd.Function):
    """out[t] = sum_k weights[t,k] * y[row(t,k)]; backward gives dY and dWeights."""

    @staticmethod
    def forward(ctx, y_RD, weights_TK, plan, round_terms):
        ctx.save_for_backward(y_RD, weights_TK)
        ctx.plan = plan
        return ops.combine_fwd(y_RD, weights_TK, plan, round_terms)

    @staticmethod
    @once_differentiable
    def backward(ctx, dout):
        y, w = ctx.saved_tensors
        dy, dw = ops.combine_bwd(dout, y, w, ctx.plan)
        return dy, dw.to(w.dtype), None, None


def router_gate(x_TD, weight_ED, logit_bias_E=None):
    return RouterGateLinearFunction.apply(x_TD, weight_ED, logit_bias_E)


def route_select(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                 num_groups=0, num_limited=0, mode=ops.SELECT_TOPK, want_scores=False):
    return RouteSelectFunction.apply(
        logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
        num_groups or 0, num_limited or 0, mode, want_scores,
    )


def route_select_cutoff(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
    return RouteSelectCutoffFunction.apply(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale)


def rms_norm(x, weight, epsilon):
    return RMSNormFunction.apply(x, weight, epsilon)


def permute_rows(x_TD, plan):
    return PermuteRowsFunction.apply(x_TD, plan)


def grouped_swiglu(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan):
    return GroupedSwiGLUFunction.apply(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan)


def gather_grouped_swiglu(x_TD, w1_EFD, w3_EFD, w2_EDF, plan):
    return GatherGroupedSwiGLUFunction.apply(x_TD, w1_EFD, w3_EFD, w2_EDF, plan)


def gather_experts_combine(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan, round_terms=True):
    return GatherExpertsCombineFunction.apply(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan, round_terms)


def combine(y_RD, weights_TK, plan, round_terms=True):
    return CombineFunction.apply(y_RD, weights_TK, plan, round_terms)
