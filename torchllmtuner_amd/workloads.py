"""The five synthetic workloads the block is measured and tested on, built from the product's
own modules: shapes, router settings, seeded random weights and inputs.

  c1  tiny Qwen3-MoE-style block, fp32, T=512 (2 x 256), D=256, E=8, F=512, softmax top-2 + norm,
      forward + backward
  c2  Qwen3-30B-A3B-shaped layer, bf16, T=8192, D=2048, E=128, K=8, F=768, forward only
  c3  the same, forward + backward (every gradient)
  c4  the same shape at T=16384 with skewed routing: a per-expert logit bias of Zipf(1.2) shape,
      scaled so that the top 20 % of the experts receive 60 % of the assignments; expert segments
      padded to 128 rows; forward + backward
  c5  DeepSeek-V3-shaped routing with one GPU's expert share: D=7168, E=256, sigmoid scores +
      expert bias ~ U(-0.1, 0.1), 8 groups / 4 kept, top-8, scale 2.5, F=2048, T=4096, experts
      0-31 computed here (the other assignments only counted), one shared expert of width 2048;
      forward + backward

Weights ~ N(0, 0.02), tokens and output gradients ~ N(0, 1), all from seeded CPU generators
(the router weight stays fp32 under bf16 experts, as the reference keeps it).
"""

from __future__ import annotations

from dataclasses import dataclass

import torch

from . import moe


@dataclass(frozen=True)
class Workload:
    key: str
    name: str
    tokens: int
    dim: int
    num_experts: int
    top_k: int
    hidden_dim: int
    dtype: torch.dtype = torch.bfloat16
    score_func: str = "softmax"
    route_norm: bool = True
    route_scale: float = 1.0
    num_expert_groups: int | None = None
    num_limited_groups: int | None = None
    backward: bool = True
    pad_multiple: int | None = None           # padded dispatch (c4)
    local_experts: tuple[int, int] | None = None  # one rank's share (c5)
    shared_hidden_dim: int | None = None
    expert_bias: bool = False                 # aux-loss-free bias ~ U(-0.1, 0.1)
    zipf_top20_share: float | None = None     # skewed routing through a router logit bias
    batch_shape: tuple[int, ...] | None = None

    @property
    def num_local_experts(self) -> int:
        lo, hi = self.local_experts or (0, self.num_experts)
        return hi - lo


WORKLOADS = {
    "c1": Workload("c1", "tiny-qwen3-moe block fwd+bwd T=512 fp32", 512, 256, 8, 2, 512, dtype=torch.float32,
                   batch_shape=(2, 256)),
    "c2": Workload("c2", "qwen3-30b-a3b-moe-layer fwd T=8192 bf16", 8192, 2048, 128, 8, 768, backward=False),
    "c3": Workload("c3", "qwen3-30b-a3b-moe-layer fwd+bwd T=8192 bf16", 8192, 2048, 128, 8, 768),
    "c4": Workload("c4", "qwen3-30b-a3b-moe-layer fwd+bwd T=16384 bf16 zipf(1.2)-skewed, 128-row padded segments",
                   16384, 2048, 128, 8, 768, pad_multiple=128, zipf_top20_share=0.60),
    "c5": Workload("c5", "deepseek-v3-moe-layer fwd+bwd T=4096 bf16, experts 0-31 of 256 local, shared expert",
                   4096, 7168, 256, 8, 2048, score_func="sigmoid", route_scale=2.5, num_expert_groups=8,
                   num_limited_groups=4, local_experts=(0, 32), shared_hidden_dim=2048, expert_bias=True),
}


def zipf_logit_bias(logits_TE: torch.Tensor, top_k: int, *, exponent: float = 1.2,
                    top20_share: float = 0.60, iters: int = 40):
    """A per-expert logit bias ``-a * exponent * ln(rank)`` (expert 0 the most popular), with the
    strength ``a`` solved by bisection so that, over the given (unbiased) logits, the busiest fifth
    of the experts receives ``top20_share`` of the top-k assignments.  Returns ``(bias_E, share)``
    with the share actually reached on those logits."""
    E = logits_TE.shape[1]
    shape = -exponent * torch.log(torch.arange(1, E + 1, dtype=torch.float32, device=logits_TE.device))
    fifth = max(E // 5, 1)
    logits = logits_TE.float()

    def share(a: float) -> float:
        ids = torch.topk(logits + a * shape, top_k, dim=-1).indices
        counts = torch.bincount(ids.reshape(-1), minlength=E).sort(descending=True).values
        return float(counts[:fifth].sum()) / ids.numel()

    lo, hi = 0.0, 1.0
    while share(hi) < top20_share and hi < 64.0:
        hi *= 2.0
    for _ in range(iters):
        mid = 0.5 * (lo + hi)
        if share(mid) < top20_share:
            lo = mid
        else:
            hi = mid
    return hi * shape, share(hi)


def make_weights(wl: Workload, seed: int = 0, std: float = 0.02) -> dict[str, torch.Tensor]:
    """Seeded CPU tensors: router (E, D) fp32; w1, w3 (El, F, D), w2 (El, D, F) and the shared
    expert's gate / up (Fs, D), down (D, Fs) in the workload's dtype."""
    g = torch.Generator().manual_seed(seed)
    D, E, F, El = wl.dim, wl.num_experts, wl.hidden_dim, wl.num_local_experts
    rnd = lambda *shape: torch.randn(*shape, generator=g) * std
    w = {"router": rnd(E, D), "w1": rnd(El, F, D).to(wl.dtype), "w3": rnd(El, F, D).to(wl.dtype),
         "w2": rnd(El, D, F).to(wl.dtype)}
    if wl.shared_hidden_dim:
        Fs = wl.shared_hidden_dim
        w.update(shared_gate=rnd(Fs, D).to(wl.dtype), shared_up=rnd(Fs, D).to(wl.dtype),
                 shared_down=rnd(D, Fs).to(wl.dtype))
    if wl.expert_bias:
        w["expert_bias"] = torch.rand(E, generator=torch.Generator().manual_seed(2)) * 0.2 - 0.1
    return w


def make_inputs(wl: Workload, seed_x: int = 0, seed_grad: int = 1):
    """(tokens, output gradient), CPU, in the workload's dtype and batch shape."""
    shape = (*(wl.batch_shape or (wl.tokens,)), wl.dim)
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(seed_x)).to(wl.dtype)
    gout = torch.randn(*shape, generator=torch.Generator().manual_seed(seed_grad)).to(wl.dtype)
    return x, gout


def build_block(wl: Workload, device, weights: dict[str, torch.Tensor] | None = None, *,
                x_for_skew: torch.Tensor | None = None) -> moe.MoE:
    """The MoE block of a workload on ``device``, holding ``weights`` (default: ``make_weights``).

    For a skewed workload the router gate carries the solved logit bias (as ``router.gate.bias``,
    llmtuner/models/common/linear.py:181-182); ``x_for_skew`` are the tokens it is solved on
    (default: the workload's own inputs).  The reached top-20 % share is left in
    ``block.skew_top20_share``."""
    w = weights if weights is not None else make_weights(wl)
    D, E, K, F = wl.dim, wl.num_experts, wl.top_k, wl.hidden_dim
    router = moe.TokenChoiceTopKRouter(
        E, D, K, score_func=wl.score_func, route_norm=wl.route_norm, route_scale=wl.route_scale,
        num_expert_groups=wl.num_expert_groups, num_limited_groups=wl.num_limited_groups)
    if wl.pad_multiple:
        dispatcher = moe.PaddedTokenDispatcher(E, K, pad_multiple=wl.pad_multiple)
    elif wl.local_experts:
        lo, hi = wl.local_experts
        dispatcher = moe.LocalShareTokenDispatcher(E, K, local_start=lo, num_local_experts=hi - lo)
    else:
        dispatcher = moe.LocalTokenDispatcher(E, K)
    shared = moe.DenseSwiGLU(D, wl.shared_hidden_dim) if wl.shared_hidden_dim else None
    block = moe.MoE(E, moe.RoutedExperts(moe.GroupedExperts(D, F, wl.num_local_experts), dispatcher), router,
                    load_balance_coeff=1e-3 if wl.expert_bias else None, shared_experts=shared)
    block = block.to(wl.dtype)
    block.router.gate.float()  # the router stays fp32 under bf16 experts (block_conversion.py:247-249)
    with torch.no_grad():
        block.router.gate.weight.copy_(w["router"])
        ie = block.routed_experts.inner_experts
        ie.w1_EFD.copy_(w["w1"]); ie.w3_EFD.copy_(w["w3"]); ie.w2_EDF.copy_(w["w2"])
        if shared is not None:
            shared.gate_proj.weight.copy_(w["shared_gate"])
            shared.up_proj.weight.copy_(w["shared_up"])
            shared.down_proj.weight.copy_(w["shared_down"])
        if wl.expert_bias:
            block.expert_bias_E.copy_(w["expert_bias"])
    if wl.zipf_top20_share:
        if "router_bias" in w:
            bias, reached = w["router_bias"], float("nan")
        else:
            x = x_for_skew if x_for_skew is not None else make_inputs(wl)[0]
            sample = x.reshape(-1, D)[:4096].float()
            bias, reached = zipf_logit_bias(sample @ w["router"].float().T, K, top20_share=wl.zipf_top20_share)
        block.router.gate.bias = torch.nn.Parameter(bias.clone().float(), requires_grad=False)
        block.skew_top20_share = reached
    return block.to(device)


def flops_per_step(wl: Workload, routed_rows: int) -> float:
    """Algorithmic FLOPs of the expert GEMMs in one step (the reference's convention,
    llmtuner/utils/flops.py:81-86,320-331: 2*R*D*F per projection over real rows only; three
    projections forward, twice that backward), shared expert included."""
    per_pass = 3 if not wl.backward else 9
    flops = 2.0 * routed_rows * wl.dim * wl.hidden_dim * per_pass
    if wl.shared_hidden_dim:
        flops += 2.0 * wl.tokens * wl.dim * wl.shared_hidden_dim * per_pass
    return flops


def describe(wl: Workload) -> dict:
    d = {"workload": wl.name, "tokens": wl.tokens, "hidden": wl.dim, "experts": wl.num_experts, "top_k": wl.top_k,
         "moe_intermediate": wl.hidden_dim, "pass": "fwd+bwd" if wl.backward else "fwd",
         "router": f"fp32 {wl.score_func} top-{wl.top_k}" + (", norm_topk_prob" if wl.route_norm else "")
                   + (f", scale {wl.route_scale}" if wl.route_scale != 1.0 else "")
                   + (f", {wl.num_expert_groups} groups / {wl.num_limited_groups} kept" if wl.num_expert_groups else "")
                   + (", expert bias U(-0.1,0.1)" if wl.expert_bias else "")}
    if wl.pad_multiple:
        d["padded_segments"] = wl.pad_multiple
    if wl.zipf_top20_share:
        d["skew"] = f"logit bias -a*1.2*ln(rank), a solved for a top-20% load share of {wl.zipf_top20_share}"
    if wl.local_experts:
        d["local_experts"] = list(wl.local_experts)
    if wl.shared_hidden_dim:
        d["shared_expert_intermediate"] = wl.shared_hidden_dim
    return d


__all__ = ["WORKLOADS", "Workload", "build_block", "describe", "flops_per_step", "make_inputs", "make_weights",
           "zipf_logit_bias"]
