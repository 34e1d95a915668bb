"""Differentiable stages of the MoE block, one function per stage.

Each function is a ``mi355_moe`` torch.library operator with its autograd formula
registered next to it (``torchllmtuner_amd/ops.py``): the backward of every stage is the
hand-written kernel for that stage, nothing here falls back to PyTorch math, and the
operators trace under ``torch.compile``.  Stages (the reference lines each replaces are
cited in include/mi355_moe.h):

  router_gate              logits = x . W^T in fp32                (custom fwd + bwd GEMMs)
  route_select             scores -> top-k -> gather -> norm       (fused select, fused VJP)
  permute_rows             expert-major row gather                 (bwd: K-way row sum)
  grouped_swiglu           gate/up/SiLU*mul/down grouped GEMMs     (bwd: dX and dW GEMMs)
  combine                  weighted unpermute                      (bwd: dY and dScore)
  gather_experts_combine   permute + experts + combine in one node: the row gather rides in
                           the GEMM operand loads, the combine's backward in the dH epilogue
"""

from __future__ import annotations

from . import ops


def router_gate(x_TD, weight_ED, logit_bias_E=None):
    """Router projection with fp32 output and fp32 backward GEMMs
    (llmtuner/models/common/linear.py:103-151: ``dX`` comes back in the input dtype and
    ``dW`` in the weight dtype)."""
    return ops.router_gate_fwd(x_TD, weight_ED, logit_bias_E)


def route_select(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                 num_groups=0, num_limited=0, mode=ops.SELECT_TOPK, want_scores=False, want_map=False):
    """Fused score function, expert choice, gather, norm and scale.

    Returns ``(weights_TK, ids_TK, scores_TE or None)`` (plus the bool routing map with
    ``want_map``).  ``scores_TE`` is only materialised (and differentiable) when
    ``want_scores`` is set, which is what an auxiliary loss on the full score map needs."""
    return ops.router_select_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale,
                                 num_groups or 0, num_limited or 0, mode, want_scores, want_map)


def route_select_cutoff(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale):
    """The same selection for a quantile-balanced router in training: also returns the dense
    score map and the (K+1)-th biased score of every token (not differentiable; it only feeds
    the required-bias histogram).  Returns ``(weights_TK, ids_TK, scores_TE, cutoff_T)``."""
    return ops.router_select_cutoff_fwd(logits_TE, expert_bias_E, top_k, score_func, route_norm, route_scale)


def rms_norm(x, weight, epsilon):
    """y = x * rsqrt(mean(x^2) + eps) * weight over the last axis; keeps only rstd."""
    return ops.rms_norm_fwd(x, weight, epsilon)[0]


def permute_rows(x_TD, plan):
    """rows[r] = x[token of row r]; backward sums the K row gradients per token."""
    return ops.permute_rows_fwd(x_TD, plan)


def grouped_swiglu(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan, zero_fill=False):
    """y = (silu(rows.w1^T) * rows.w3^T) . w2^T per expert segment."""
    return ops.grouped_swiglu_fwd(rows_RD, w1_EFD, w3_EFD, w2_EDF, plan, zero_fill=zero_fill)[0]


def gather_experts_combine(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan, round_terms=True):
    """out[t] = sum_k weights[t,k] * experts(x)[row(t,k)] with one backward for both halves."""
    return ops.gather_experts_combine(x_TD, weights_TK, w1_EFD, w3_EFD, w2_EDF, plan, round_terms)


def combine(y_RD, weights_TK, plan, round_terms=True):
    """out[t] = sum_k weights[t,k] * y[row(t,k)]; backward gives dY and dWeights."""
    return ops.combine_fwd(y_RD, weights_TK, plan, round_terms)
