"""Shared helpers for the parity tests: seeded inputs, error metrics, fragility."""

from __future__ import annotations

import torch

from oracle import moe_ref as R


# Lines for the end-of-run summary (tests/conftest.py prints them whatever the verbosity): how
# many tokens differed from the oracle, load histograms -- figures a passing test would hide.
PARITY_NOTES: list[str] = []


def note(line: str) -> None:
    print(line, flush=True)
    PARITY_NOTES.append(line)


def rel_l2(a: torch.Tensor, b: torch.Tensor) -> float:
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    return float((a - b).norm() / b.norm().clamp_min(1e-30))


def rel_max(a: torch.Tensor, b: torch.Tensor) -> float:
    """max |a-b| relative to the reference's largest magnitude."""
    a, b = a.detach().double().cpu(), b.detach().double().cpu()
    if b.numel() == 0:
        return 0.0
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


def stable_tokens(logits_TE, spec: R.RouterSpec, expert_bias_E=None, trials=4, eps=2e-6):
    """Tokens whose routing decision (ids AND their order) survives relative
    perturbations of the scores of size ``eps`` -- i.e. is not decided by a few ulps
    of exp/sigmoid.  Everything outside this mask is a near tie where bit-exact
    agreement between two correct implementations is not defined."""
    base = R.score(logits_TE, spec.score_func)
    ref = R.select_experts(base, expert_bias_E, spec.top_k, spec.num_expert_groups, spec.num_limited_groups)
    ok = torch.ones(logits_TE.shape[0], dtype=torch.bool)
    g = torch.Generator().manual_seed(1234)
    for _ in range(trials):
        noise = 1.0 + eps * (2 * torch.rand(base.shape, generator=g) - 1)
        ids = R.select_experts(base * noise, expert_bias_E, spec.top_k, spec.num_expert_groups, spec.num_limited_groups)
        ok &= (ids == ref).all(dim=-1)
    return ok


def exact_score_ties(logits_TE, spec: R.RouterSpec, expert_bias_E=None):
    """Tokens whose K+1 best choice scores (oracle arithmetic, fp32) contain two EQUAL values:
    there the reference's ``torch.topk`` may pick either expert, and so may any correct
    implementation.  Everywhere else the selection -- ids and their order -- is determined."""
    s = R.score(logits_TE, spec.score_func)
    c = s if expert_bias_E is None else s + expert_bias_E
    top = torch.topk(c, min(spec.top_k + 1, c.shape[-1]), dim=-1).values
    return (top[:, 1:] == top[:, :-1]).any(-1)


def make_params(E, D, F, dtype, seed=0, std=0.02, shared_F=None, El=None):
    """N(0, std) weights from a seeded CPU generator; router weight stays fp32."""
    g = torch.Generator().manual_seed(seed)
    El = E if El is None else El
    p = R.MoEParams(
        router_w_ED=torch.randn(E, D, generator=g) * std,
        w1_EFD=(torch.randn(El, F, D, generator=g) * std).to(dtype),
        w3_EFD=(torch.randn(El, F, D, generator=g) * std).to(dtype),
        w2_EDF=(torch.randn(El, D, F, generator=g) * std).to(dtype),
    )
    if shared_F:
        p.shared_gate_FD = (torch.randn(shared_F, D, generator=g) * std).to(dtype)
        p.shared_up_FD = (torch.randn(shared_F, D, generator=g) * std).to(dtype)
        p.shared_down_DF = (torch.randn(D, shared_F, generator=g) * std).to(dtype)
    return p


def build_block(p: R.MoEParams, spec: R.RouterSpec, D, F, dtype, device, *, dispatcher="local",
                pad_multiple=None, local=None, load_balance_coeff=None, activation=None):
    """The device MoE block holding exactly the oracle's parameters."""
    from torchllmtuner_amd import moe

    E, K = spec.num_experts, spec.top_k
    El = p.w1_EFD.shape[0]
    router = moe.TokenChoiceTopKRouter(
        E, D, K, score_func=spec.score_func, route_norm=spec.route_norm, route_scale=spec.route_scale,
        num_expert_groups=spec.num_expert_groups, num_limited_groups=spec.num_limited_groups,
        fixed_router=spec.fixed_router, _debug_force_load_balance=spec.debug_force_load_balance,
    )
    if dispatcher == "padded":
        disp = moe.PaddedTokenDispatcher(E, K, pad_multiple=pad_multiple)
    elif dispatcher == "share":
        disp = moe.LocalShareTokenDispatcher(E, K, local_start=local[0], num_local_experts=local[1] - local[0])
    else:
        disp = moe.LocalTokenDispatcher(E, K)
    shared = None
    if p.shared_gate_FD is not None:
        shared = moe.DenseSwiGLU(D, p.shared_gate_FD.shape[0])
    block = moe.MoE(E, moe.RoutedExperts(moe.GroupedExperts(D, F, El, activation_fn=activation), disp), router,
                    load_balance_coeff=load_balance_coeff, shared_experts=shared)
    block = block.to(dtype)
    block.router.gate.float()  # router stays fp32 under bf16 experts
    with torch.no_grad():
        block.router.gate.weight.copy_(p.router_w_ED)
        ie = block.routed_experts.inner_experts
        ie.w1_EFD.copy_(p.w1_EFD); ie.w3_EFD.copy_(p.w3_EFD); ie.w2_EDF.copy_(p.w2_EDF)
        if shared is not None:
            shared.gate_proj.weight.copy_(p.shared_gate_FD)
            shared.up_proj.weight.copy_(p.shared_up_FD)
            shared.down_proj.weight.copy_(p.shared_down_DF)
        if p.expert_bias_E is not None:
            block.expert_bias_E.copy_(p.expert_bias_E)
    if p.router_logit_bias_E is not None:  # carried as router.gate.bias (linear.py:181-182)
        block.router.gate.bias = torch.nn.Parameter(p.router_logit_bias_E.clone(), requires_grad=False)
    return block.to(device)
