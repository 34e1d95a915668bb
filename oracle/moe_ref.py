"""CPU restatement of TorchLLMTuner's native MoE block -- TEST INFRASTRUCTURE ONLY.

This module is the parity oracle for the MI355X kernels.  It is imported only by
``tests/``, by ``__graft_entry__.smoke()`` and by the ``cpu_baseline`` leg of
``bench.py``; nothing in ``torchllmtuner_amd`` may import it, and the product
path never falls back to it.

Every function restates one step of the reference block with stock PyTorch CPU
ops, keeping the reference's op order and dtype rounding points, and cites the
reference lines it follows (paths relative to the reference checkout).  Backward
comes from autograd, exactly as in the reference (its only hand-written backward
is the router gate's, restated in ``RouterGateFn``).

One deliberate, documented difference: ``torch.topk(sorted=False)`` leaves both
the tie winner and the within-row order unspecified.  The oracle fixes the
canonical rule "higher score first, ties to the lower expert index" by a stable
descending sort; per-row *sets* equal ``torch.topk``'s whenever no tie straddles
the K-th boundary (checked in tests/test_oracle.py).

Pinning status (tests/test_oracle.py holds the checks):
  router_gate            pinned: equals a plain fp32 linear bit-for-bit; fp64 literals
  score/select/route     pinned: closed forms, set-equality with torch.topk, literals
  select_within_groups   pinned: known answer ids [[0,1]], confinement invariant
  fixed/balanced routing pinned: closed forms (t+k)%E, (t*K+k)%E, weights 1/K
  local_reorder/permute  pinned: known answer rows [0,1,1,2,0,2] + duplicate-row VJP
  permute_and_pad        pinned: invariants padded=c+(-c%m), rows==sum(padded),
                         equality with the local path after combine, analytic 2*sum(w)
  grouped_experts        pinned: per-segment hand reference, zero-count segments fp64
  situ_glu               pinned: the explicit formula of the reference's own test
                         (tests/unit_tests/cpu/models/test_situ_activation.py:31-45) for
                         linear_beta None / 0 / 1.7, values and gradients; |out| <= beta*|up|
                         and the small-argument limit gate*up/2
  combine                pinned: inverse-permute/reshape/sum reference, fp64 exactness
  moe_forward            pinned: analytic experts x(id+1), brute-force fp64 loop
  balance_loss           pinned: the paper formula, even-load value, scale and order invariance
  select_top_k_plus_one, quantile_observe, quantile_estimate
                         pinned: the reference's worked example (bins 1/3/5/6, next bias
                         [-0.55,-0.15,0.25,0.45]), its past-int32 and fractional-large-count
                         literals, empty-window identity, mean-centring, padding filter,
                         pair-by-pair brute force
  rms_norm               pinned: the reference's fp64 formula + gradcheck, and bit-equality
                         with torch.nn.functional.rms_norm (the reference's CPU backend) in
                         fp32 and bf16
  local-share (experts [lo,hi) only)  parity unpinned against the reference: the
                         reference has no single-process form of "one EP rank's
                         share"; defined here as dropping the sorted rows outside
                         the local expert range and pinned only by brute force.
"""

from __future__ import annotations

from dataclasses import dataclass

import torch
import torch.nn.functional as F

__all__ = [
    "RouterGateFn",
    "router_gate",
    "score",
    "select_experts",
    "select_experts_within_groups",
    "route",
    "routing_map",
    "local_reorder",
    "permute_and_pad",
    "unpermute_padded",
    "grouped_experts",
    "situ_glu",
    "combine",
    "shared_expert",
    "balance_loss",
    "select_top_k_plus_one",
    "quantile_observe",
    "quantile_estimate",
    "rms_norm",
    "moe_forward",
    "MoEParams",
    "RouterSpec",
]


# --------------------------------------------------------------------------
# router gate: llmtuner/models/common/linear.py:103-151, 179-183
# --------------------------------------------------------------------------
class RouterGateFn(torch.autograd.Function):
    """fp32 forward GEMM and fp32 backward GEMMs whatever the storage dtype.

    Follows ``RouterGateLinearFunction`` (linear.py:107-151), portable branch
    (:124-127): operands are promoted with ``.float()``; ``dX`` is cast back to
    the input dtype and ``dW`` to the weight dtype.
    """

    @staticmethod
    def forward(ctx, x_TD, w_ED):
        x32 = x_TD.float()
        w32 = w_ED.float()
        ctx.save_for_backward(x32, w32)
        ctx.in_dtype = x_TD.dtype
        ctx.w_dtype = w_ED.dtype
        return torch.mm(x32, w32.T)

    @staticmethod
    def backward(ctx, g_TE):
        x32, w32 = ctx.saved_tensors
        g32 = g_TE.float()
        gx = torch.mm(g32, w32).to(ctx.in_dtype) if ctx.needs_input_grad[0] else None
        gw = torch.mm(g32.T, x32).to(ctx.w_dtype) if ctx.needs_input_grad[1] else None
        return gx, gw


def router_gate(x_TD, w_ED, logit_bias_E=None):
    """``RouterGateLinear.forward`` (linear.py:179-183): logits + optional fp32 bias."""
    out = RouterGateFn.apply(x_TD, w_ED)
    if logit_bias_E is not None:
        out = out + logit_bias_E.float()
    return out


# --------------------------------------------------------------------------
# scores and selection: llmtuner/models/common/moe/routing.py:168-239, 266-324
# --------------------------------------------------------------------------
def score(logits_TE, score_func):
    """routing.py:270-277."""
    if score_func == "sigmoid":
        return torch.sigmoid(logits_TE)
    if score_func == "softmax":
        return F.softmax(logits_TE, dim=-1)
    if score_func == "sqrtsoftplus":
        return F.softplus(logits_TE).sqrt()
    raise NotImplementedError(f"Unknown score function {score_func}")


def _topk_lower_index_ties(values, k):
    """Indices of the k largest entries per row; ties go to the lower index.

    Canonical replacement for ``torch.topk(..., sorted=False).indices``
    (routing.py:189-191): a stable descending sort keeps equal values in
    ascending index order, so the first k are "largest, lowest index first".
    """
    return torch.sort(values, dim=-1, descending=True, stable=True).indices[..., :k]


def _topk_values_lower_index_ties(values, k):
    return torch.sort(values, dim=-1, descending=True, stable=True).values[..., :k]


def select_experts_within_groups(choice_TE, top_k, num_groups, num_limited):
    """routing.py:194-239: group score = sum of top-2, keep top-L groups, -inf mask."""
    T, E = choice_TE.shape
    P = E // num_groups
    s_TGP = choice_TE.unflatten(-1, (num_groups, P))
    group_TG = _topk_values_lower_index_ties(s_TGP, 2).sum(dim=-1)
    sel_TL = _topk_lower_index_ties(group_TG, num_limited)
    unselected_TG = torch.ones_like(group_TG, dtype=torch.bool)
    unselected_TG.scatter_(-1, sel_TL, False)
    masked_TE = s_TGP.masked_fill(unselected_TG.unsqueeze(-1), float("-inf")).flatten(-2)
    return _topk_lower_index_ties(masked_TE, top_k)


def select_experts(scores_TE, expert_bias_E, top_k, num_groups=None, num_limited=None):
    """routing.py:168-192: the bias steers the choice only."""
    choice = scores_TE if expert_bias_E is None else scores_TE + expert_bias_E
    if num_groups is None:
        return _topk_lower_index_ties(choice, top_k)
    return select_experts_within_groups(choice, top_k, num_groups, num_limited)


@dataclass
class RouterSpec:
    """The router's constructor surface (routing.py:64-78), minus the aux loss."""

    num_experts: int
    top_k: int
    score_func: str = "sigmoid"
    route_norm: bool = False
    route_scale: float = 1.0
    num_expert_groups: int | None = None
    num_limited_groups: int | None = None
    fixed_router: bool = False
    debug_force_load_balance: bool = False


def route(logits_TE, spec: RouterSpec, expert_bias_E=None):
    """``TokenChoiceTopKRouter.forward`` after the gate (routing.py:270-345).

    Returns ``(topk_scores_TK fp32, topk_ids_TK int64, routing_map_TE bool)``.
    """
    scores_TE = score(logits_TE, spec.score_func)
    T = scores_TE.shape[0]
    K, E = spec.top_k, spec.num_experts
    if spec.fixed_router:  # routing.py:291-295
        ids = (torch.arange(T)[:, None] + torch.arange(K)[None, :]) % E
    elif spec.debug_force_load_balance:  # routing.py:146-166
        ids = torch.arange(T * K, dtype=torch.int64).reshape(T, K) % E
    else:
        ids = select_experts(
            scores_TE, expert_bias_E, K, spec.num_expert_groups, spec.num_limited_groups
        )
    if spec.fixed_router:  # routing.py:304-309
        w = scores_TE.new_full(ids.shape, 1.0 / K)
    else:  # routing.py:311-315
        w = scores_TE.gather(dim=-1, index=ids)
        if spec.route_norm:
            w = w / (w.sum(dim=-1, keepdim=True) + 1e-20)
        w = w * spec.route_scale
    return w, ids, routing_map(ids, E)


def routing_map(ids_TK, num_experts):
    """routing.py:320-324: one-hot by scatter (a repeated id still counts once)."""
    m = torch.zeros(ids_TK.shape[0], num_experts, dtype=torch.bool)
    return m.scatter_(-1, ids_TK, True)


# --------------------------------------------------------------------------
# dispatch: llmtuner/parallel/expert_parallel/token_dispatch.py:146-199
# --------------------------------------------------------------------------
def local_reorder(x_TD, scores_TK, ids_TK):
    """token_dispatch.py:180-199: stable argsort by expert, gather rows.

    Returns ``(rows_ND, token_index_N int64, scores_sorted_N, perm_N int64)``.
    """
    K = ids_TK.shape[1]
    perm = torch.argsort(ids_TK.reshape(-1), stable=True)
    s_sorted = scores_TK.reshape(-1)[perm]
    tok = perm // K
    return x_TD[tok], tok, s_sorted, perm


def permute_and_pad(rows_RD, counts_E, pad_multiple):
    """Padded expert-major layout used by ``TorchAOTokenDispatcher`` at EP=1.

    Restates the executable contract at
    tests/unit_tests/cpu/models/test_moe_token_dispatch.py:154-179 (the
    reference's stand-in for torchao's ``permute_and_pad``; the real torchao
    kernel is absent from the reference tree, so its treatment of zero-count
    experts is *parity unpinned* -- here they get no padding rows because
    ``-0 % m == 0``).  Returns ``(ext_shape, padded_rows, permuted_indices,
    padded_counts)``; padding rows point at a zero sentinel row of index R.
    """
    R, D = rows_RD.shape
    counts = [int(c) for c in counts_E.tolist()]
    ext = torch.cat([rows_RD, rows_RD.new_zeros(1, D)], dim=0)
    idx: list[int] = []
    pos = 0
    for c in counts:
        idx.extend(range(pos, pos + c))
        idx.extend([R] * (-c % pad_multiple))
        pos += c
    assert pos == R
    idx_t = torch.tensor(idx, dtype=torch.long)
    padded = torch.tensor([c + (-c % pad_multiple) for c in counts], dtype=torch.long)
    return ext.shape, ext[idx_t], idx_t, padded


def unpermute_padded(rows_PD, ext_shape, permuted_indices):
    """token_dispatch.py:626-635 + torchao_dispatch.py:177-185: strip the padding."""
    out = rows_PD.new_empty(ext_shape)
    out[permuted_indices, :] = rows_PD
    return out[: ext_shape[0] - 1]


# --------------------------------------------------------------------------
# experts: llmtuner/models/common/moe/experts.py:152-285, activation.py:33-37
# --------------------------------------------------------------------------
def _segment_linear(x_RI, w_EOI, counts):
    """The per-expert loop of ``_grouped_mm`` (experts.py:272-285)."""
    if x_RI.shape[0] == 0:  # experts.py:229-233
        return F.linear(x_RI, w_EOI[0].to(x_RI.dtype))
    out = x_RI.new_empty(x_RI.shape[0], w_EOI.shape[1])
    start = 0
    for e, c in enumerate(counts):
        out[start : start + c] = F.linear(x_RI[start : start + c], w_EOI[e])
        start += c
    return out


def situ_glu(gate, up, beta=1.0, linear_beta=None):
    """``SituGLU.forward`` (activation.py:58-64): fp32 arithmetic, result in the gate's dtype."""
    g, u = gate.float(), up.float()
    act = beta * torch.tanh(g / beta) * g.sigmoid()
    if linear_beta not in (None, 0.0):
        u = linear_beta * torch.tanh(u / linear_beta)
    return (act * u).to(gate.dtype)


def grouped_experts(x_RD, counts_E, w1_EFD, w3_EFD, w2_EDF, activation=None):
    """``GroupedExperts._compute`` (experts.py:204-209) on the loop path.

    gate, up and the activation's product are each materialised in the activation
    dtype, which is where the reference's bf16 rounding points are.  ``activation``
    is the ``(gate, up)`` function of experts.py:207; None is SwiGLU.
    """
    counts = [int(c) for c in counts_E.tolist()]
    assert sum(counts) == x_RD.shape[0]
    gate = _segment_linear(x_RD, w1_EFD, counts)
    up = _segment_linear(x_RD, w3_EFD, counts)
    if activation is None:
        h = F.silu(gate) * up  # activation.py:36-37
    else:
        h = activation(gate, up)
    return _segment_linear(h, w2_EDF, counts).type_as(x_RD)


# --------------------------------------------------------------------------
# combine: token_dispatch.py:234-275
# --------------------------------------------------------------------------
def combine(y_RD, tok_R, s_sorted_R, x_TD, accumulate_in_fp32=False):
    """fp32 score multiply, cast, ``index_add`` by token, cast to x dtype."""
    compute_dtype = torch.promote_types(y_RD.dtype, torch.float32)
    acc_dtype = compute_dtype if accumulate_in_fp32 else y_RD.dtype
    out = torch.zeros_like(x_TD, dtype=compute_dtype if accumulate_in_fp32 else x_TD.dtype)
    weighted = (y_RD.to(compute_dtype) * s_sorted_R.reshape(-1, 1)).to(acc_dtype)
    out = out.index_add(0, tok_R, weighted)
    return out.to(x_TD.dtype)


def balance_loss(scores_TE, routing_map_TE, padding_mask_T=None):
    """``MicrobatchWiseLoadBalanceLoss.forward`` up to ``inject``
    (llmtuner/models/common/moe/auxiliary_loss.py:147-162), one process: counts from the
    (already padding-filtered) map, ``f = normalize(counts, p=1) * E``, per-token
    L1-normalised scores with padding rows zeroed, ``loss = sum f * p``."""
    import torch.nn.functional as F

    counts_E = routing_map_TE.to(scores_TE.dtype).sum(dim=0)
    f_E = F.normalize(counts_E, p=1, dim=0) * scores_TE.size(-1)
    probs_TE = F.normalize(scores_TE, p=1, dim=-1)
    if padding_mask_T is not None:
        probs_TE = probs_TE * ~padding_mask_T.unsqueeze(-1)
    p_E = probs_TE.sum(dim=0)
    return (f_E * p_E).sum()


def select_top_k_plus_one(scores_TE, expert_bias_E, top_k):
    """Training-time selection of the quantile-balanced router
    (llmtuner/models/common/moe/routing.py:411-430): one sorted top-(K+1) over the biased
    scores; the first K ids route, the (K+1)-th biased score is the cutoff.  Ties go to the
    lower expert id (stable descending sort; ``torch.topk`` leaves them unspecified).
    Returns ``(ids_TK int64, cutoff_T1 fp32)``."""
    biased_TE = scores_TE + expert_bias_E
    order = torch.argsort(biased_TE, dim=-1, descending=True, stable=True)
    cutoff_T1 = biased_TE.gather(-1, order[:, top_k:top_k + 1])
    return order[:, :top_k].contiguous(), cutoff_T1


def quantile_observe(histogram_EB, scores_TE, cutoff_T1, expert_bias_E, padding_mask_T=None):
    """``_observe_quantile_histogram`` (routing.py:433-461), in place on the int64
    histogram: required bias ``cutoff - score`` of every valid (token, expert) pair, binned
    uniformly over ``[min(bias) - 1, max(bias) + 1]``; fp32 operations in the reference's
    order, counted pair by pair."""
    if padding_mask_T is not None:
        keep = ~padding_mask_T
        scores_TE, cutoff_T1 = scores_TE[keep], cutoff_T1[keep]
    num_bins = histogram_EB.shape[1]
    lower = expert_bias_E.min() - 1.0
    width = (expert_bias_E.max() - expert_bias_E.min() + 2.0) / num_bins
    bins_TE = torch.floor((cutoff_T1 - scores_TE - lower) / width).to(torch.int64).clamp(0, num_bins - 1)
    for e in range(histogram_EB.shape[0]):
        histogram_EB[e] += torch.bincount(bins_TE[:, e], minlength=num_bins)


def quantile_estimate(histogram_EB, expert_bias_E, top_k):
    """``QuantileBalancer.estimate_expert_bias`` (routing.py:557-610): the ``K/E`` quantile
    of each expert's histogram (target rank ``ceil(count*K/E)``; position = crossing bin +
    ``(count*K - before*E) / E / in_bin``, the numerator integral), experts without
    observations held at their current position, then mean-centred and scaled by the bin
    width.  No observation at all returns a copy of the bias."""
    E, B = histogram_EB.shape
    counts_E = histogram_EB.sum(dim=-1)
    if not bool(counts_E.any()):
        return expert_bias_E.clone()
    width = (expert_bias_E.max() - expert_bias_E.min() + 2.0) / B
    pos_E = torch.empty(E, dtype=torch.float32)
    for e in range(E):
        count = int(counts_E[e])
        if count == 0:
            pos_E[e] = (expert_bias_E[e] - (expert_bias_E.min() - 1.0)) / width
            continue
        numerator = count * top_k
        rank = -(-numerator // E)
        running = 0
        for b in range(B):
            in_bin = int(histogram_EB[e, b])
            if running + in_bin >= rank:
                break
            running += in_bin
        residual = torch.tensor(numerator - running * E, dtype=torch.int64)
        fraction = residual.float() / E / torch.tensor(float(in_bin)).clamp(min=1.0)
        pos_E[e] = torch.tensor(float(b)) + fraction
    return ((pos_E - pos_E.mean()) * width).to(expert_bias_E.dtype)


def rms_norm(hidden_states, weight, epsilon):
    """The reference's CPU backend of ``rms_norm`` (llmtuner/kernel/cpu/basic.py:17-25) is
    ``torch.nn.functional.rms_norm`` over the last axis; written out: fp32 (or wider)
    arithmetic ``(x * rsqrt(mean(x^2) + eps)) * w`` and one rounding to the input dtype at the
    end (checked bit for bit against the library routine in the tests, and against the
    reference's own formula, tests/unit_tests/cpu/kernel/test_kernel_contracts.py:100-105)."""
    wide = torch.promote_types(hidden_states.dtype, torch.float32)
    x = hidden_states.to(wide)
    r = torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + epsilon)
    return ((x * r) * weight.to(wide)).to(hidden_states.dtype)


def shared_expert(x_TD, gate_w_FD, up_w_FD, down_w_DF):
    """The HF dense MLP reused as the shared expert (block_conversion.py:278-291)."""
    return F.linear(F.silu(F.linear(x_TD, gate_w_FD)) * F.linear(x_TD, up_w_FD), down_w_DF)


# --------------------------------------------------------------------------
# whole block: llmtuner/models/common/moe/layer.py:246-309
# --------------------------------------------------------------------------
@dataclass
class MoEParams:
    router_w_ED: torch.Tensor
    w1_EFD: torch.Tensor
    w3_EFD: torch.Tensor
    w2_EDF: torch.Tensor
    expert_bias_E: torch.Tensor | None = None
    router_logit_bias_E: torch.Tensor | None = None
    shared_gate_FD: torch.Tensor | None = None
    shared_up_FD: torch.Tensor | None = None
    shared_down_DF: torch.Tensor | None = None


def moe_forward(
    x,
    p: MoEParams,
    spec: RouterSpec,
    *,
    pad_multiple: int | None = None,
    accumulate_in_fp32: bool = False,
    local_experts: tuple[int, int] | None = None,
    activation=None,
):
    """``MoE.forward`` (layer.py:268-309) at EP=1.

    ``pad_multiple`` routes through the padded permute; ``local_experts=(lo, hi)``
    computes only experts ``[lo, hi)`` (weights given for those experts only) and
    drops the other assignments from compute while still counting them.
    ``activation``: the experts' gated activation (None is SwiGLU).
    Returns ``(out, aux)`` where ``aux`` holds ids, scores, counts and the sorted
    token indices for parity checks.
    """
    restore = x.dim() > 2
    tokens = x.reshape(-1, x.shape[-1]) if restore else x
    logits = router_gate(tokens, p.router_w_ED, p.router_logit_bias_E)
    w_TK, ids_TK, map_TE = route(logits, spec, p.expert_bias_E)
    counts_E = map_TE.sum(dim=0)

    rows, tok, s_sorted, perm = local_reorder(tokens, w_TK, ids_TK)
    lo, hi = (0, spec.num_experts) if local_experts is None else local_experts
    start = int(counts_E[:lo].sum())
    stop = int(counts_E[:hi].sum())
    rows, tok_l, s_l = rows[start:stop], tok[start:stop], s_sorted[start:stop]
    local_counts = counts_E[lo:hi]
    if pad_multiple is None:
        y = grouped_experts(rows, local_counts, p.w1_EFD, p.w3_EFD, p.w2_EDF, activation)
    else:
        ext_shape, padded_rows, pidx, padded_counts = permute_and_pad(
            rows, local_counts, pad_multiple
        )
        y_pad = grouped_experts(padded_rows, padded_counts, p.w1_EFD, p.w3_EFD, p.w2_EDF, activation)
        y = unpermute_padded(y_pad, ext_shape, pidx)
    out = combine(y, tok_l, s_l, tokens, accumulate_in_fp32)
    if p.shared_gate_FD is not None:
        out = out + shared_expert(tokens, p.shared_gate_FD, p.shared_up_FD, p.shared_down_DF)
    if restore:
        out = out.reshape(*x.shape[:-1], out.shape[-1])
    aux = {
        "logits": logits,
        "scores_TK": w_TK,
        "ids_TK": ids_TK,
        "counts_E": counts_E,
        "perm_N": perm,
        "token_index_N": tok,
    }
    return out, aux
