"""GPU parity of quantile-balanced routing against the CPU oracle and the reference's own
literals (tests/unit_tests/cpu/models/test_moe_routing.py:170-298, :357-367, :430-486,
:583-592): top-(K+1) selection with its cutoff, the required-bias histogram (bit-exact
integer work), the quantile estimate, the router and MoE modules and the optimizer hook."""

import pytest
import torch

from oracle import moe_ref as R
from tests.helpers import rel_max

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops():
    from torchllmtuner_amd import ops as o

    return o


def _case(T, E, K, seed, bias_span=0.4):
    g = torch.Generator().manual_seed(seed)
    logits = torch.randn(T, E, generator=g)
    bias = (torch.rand(E, generator=g) - 0.5) * bias_span
    pad = torch.rand(T, generator=g) < 0.25
    return logits, bias, pad


@pytest.mark.parametrize("T,E,K", [(6, 4, 2), (300, 8, 2), (1000, 128, 8), (257, 256, 8), (64, 96, 60)])
def test_select_cutoff_is_the_k_plus_first_biased_score(ops, T, E, K):
    print(f"select cutoff T={T} E={E} K={K}", flush=True)
    logits, bias, _ = _case(T, E, K, seed=T + E)
    w, ids, scores, cutoff = ops.router_select_cutoff_fwd(logits.to(DEV), bias.to(DEV), K, "sigmoid", True, 2.5)
    scores, cutoff, ids, w = scores.cpu(), cutoff.cpu(), ids.cpu(), w.cpu()
    assert rel_max(scores, torch.sigmoid(logits)) < 1e-6
    # exact, from the device's own scores: sorted biased scores, ids = first K, cutoff = next
    biased = scores + bias
    order = torch.argsort(biased, dim=-1, descending=True, stable=True)
    assert torch.equal(ids, order[:, :K])
    assert torch.equal(cutoff, biased.gather(-1, order[:, K:K + 1]).squeeze(-1))
    # the oracle's selection on the same scores, and the plain kernel's ids
    ref_ids, ref_cut = R.select_top_k_plus_one(scores, bias, K)
    assert torch.equal(ids, ref_ids) and torch.equal(cutoff, ref_cut.squeeze(-1))
    w2, ids2, _ = ops.router_select_fwd(logits.to(DEV), bias.to(DEV), K, "sigmoid", True, 2.5)
    assert torch.equal(ids2.cpu(), ids) and torch.equal(w2.cpu(), w)
    # weights are the unbiased scores, normalised and scaled
    picked = scores.gather(-1, ids)
    assert rel_max(w, picked / (picked.sum(-1, keepdim=True) + 1e-20) * 2.5) < 1e-6


@pytest.mark.parametrize("T,E,K", [(300, 8, 2), (1000, 128, 8), (257, 256, 8), (64, 96, 60)])
@pytest.mark.parametrize("score_func", ["sigmoid", "softmax"])
def test_select_cutoff_without_a_bias_is_the_k_plus_first_score(ops, T, E, K, score_func):
    """No expert bias: the cutoff is still a SCORE (the (K+1)-th largest), never a logit, in both
    select kernels (E = 128 / 256 take the 16-lanes-per-token kernel, the others one wave per token)."""
    print(f"select cutoff without bias T={T} E={E} K={K} {score_func}", flush=True)
    logits, _, _ = _case(T, E, K, seed=3 * T + E)
    w, ids, scores, cutoff = ops.router_select_cutoff_fwd(logits.to(DEV), None, K, score_func, True, 1.0)
    scores, cutoff, ids = scores.cpu(), cutoff.cpu(), ids.cpu()
    ref = torch.sigmoid(logits) if score_func == "sigmoid" else torch.softmax(logits, dim=-1)
    assert rel_max(scores, ref) < 1e-5
    order = torch.argsort(scores, dim=-1, descending=True, stable=True)
    assert torch.equal(cutoff, scores.gather(-1, order[:, K:K + 1]).squeeze(-1))
    assert torch.equal(ids, order[:, :K])
    ref_ids, ref_cut = R.select_top_k_plus_one(scores, torch.zeros(E), K)
    assert torch.equal(ids, ref_ids) and torch.equal(cutoff, ref_cut.squeeze(-1))


@pytest.mark.parametrize("T,E,K,B", [(4, 4, 2, 10), (300, 8, 2, 10), (1000, 128, 8, 1000), (64, 256, 8, 37),
                                     (513, 60, 4, 5000)])
@pytest.mark.parametrize("padded", [False, True])
def test_histogram_is_bit_exact_and_accumulates(ops, T, E, K, B, padded):
    print(f"observe T={T} E={E} B={B} padded={padded}", flush=True)
    logits, bias, pad = _case(T, E, K, seed=T + B)
    scores = torch.sigmoid(logits)
    _, cutoff = R.select_top_k_plus_one(scores, bias, K)
    pad = pad if padded else None
    want = torch.zeros(E, B, dtype=torch.int64)
    got = torch.zeros(E, B, dtype=torch.int64, device=DEV)
    for _ in range(2):  # two micro-batches into the same window
        R.quantile_observe(want, scores, cutoff, bias, padding_mask_T=pad)
        ops.quantile_observe(got, scores.to(DEV), cutoff.to(DEV), bias.to(DEV),
                             None if pad is None else pad.to(DEV))
    assert torch.equal(got.cpu(), want)
    valid = T if pad is None else int((~pad).sum())
    assert int(got.sum()) == 2 * valid * E


def test_histogram_counts_past_int32(ops):
    # test_moe_routing.py:357-367
    hist = torch.zeros(2, 4, dtype=torch.int64, device=DEV)
    hist[:, 2] = torch.iinfo(torch.int32).max
    ops.quantile_observe(hist, torch.full((1, 2), 0.5, device=DEV), torch.full((1, 1), 0.5, device=DEV),
                         torch.zeros(2, device=DEV))
    assert hist[:, 2].tolist() == [2147483648, 2147483648]
    assert int(hist.sum()) == 4294967296


def test_estimate_literals(ops):
    # worked example, test_moe_routing.py:233-257
    hist = torch.zeros(4, 10, dtype=torch.int64)
    for e, b in enumerate((1, 3, 5, 6)):
        hist[e, b] = 4
    got = ops.quantile_estimate(hist.to(DEV), torch.zeros(4, device=DEV), 2)
    torch.testing.assert_close(got.cpu(), torch.tensor([-0.55, -0.15, 0.25, 0.45]))
    # fractional targets at counts float32 cannot hold, test_moe_routing.py:583-592
    hist = torch.tensor([[8388609, 1, 0, 8388609], [8388609, 0, 1, 8388608]], dtype=torch.int64)
    got = ops.quantile_estimate(hist.to(DEV), torch.zeros(2, device=DEV), 1)
    assert torch.equal(got.cpu(), torch.tensor([0.125, -0.125]))
    # an empty window hands the bias back bit for bit, in a new tensor, test_moe_routing.py:430-441
    original = torch.tensor([-0.31, -0.12, 0.17, 0.26], device=DEV)
    current = original.clone()
    for _ in range(10):
        current = ops.quantile_estimate(torch.zeros(4, 32, dtype=torch.int64, device=DEV), current, 2)
    assert torch.equal(current, original) and current.data_ptr() != original.data_ptr()


@pytest.mark.parametrize("E,K,B,seed", [(4, 2, 32, 0), (128, 8, 1000, 1), (256, 8, 100, 2), (7, 3, 65, 3), (300, 1, 64, 4)])
def test_estimate_matches_the_oracle(ops, E, K, B, seed):
    print(f"estimate E={E} K={K} B={B}", flush=True)
    g = torch.Generator().manual_seed(seed)
    hist = torch.randint(0, 50, (E, B), generator=g) * (torch.rand(E, B, generator=g) < 0.3)
    hist[seed % E] = 0                      # an expert without observations keeps its place
    hist[(seed + 1) % E, :] = 0
    hist[(seed + 1) % E, B - 1] = 7         # everything in the last bin
    bias = (torch.rand(E, generator=g) - 0.5) * 0.3
    want = R.quantile_estimate(hist, bias, K)
    got = ops.quantile_estimate(hist.to(DEV), bias.to(DEV), K).cpu()
    torch.testing.assert_close(got, want, rtol=0, atol=2e-6)
    assert abs(float(got.sum())) < 1e-4


# ------------------------------------------------------------------ modules
def _routers(E=4, D=8, K=2, **kw):
    from torchllmtuner_amd.moe import QuantileBalancedTopKRouter, TokenChoiceTopKRouter

    torch.manual_seed(0)
    base = TokenChoiceTopKRouter(E, D, K).to(DEV)
    quantile = QuantileBalancedTopKRouter(E, D, K, **kw).to(DEV)
    with torch.no_grad():
        quantile.gate.weight.copy_(base.gate.weight)
    return base, quantile


def test_a_training_forward_routes_like_the_base_router_but_observes():
    # test_moe_routing.py:185-208
    base, quantile = _routers()
    base.train(); quantile.train()
    x = torch.randn(8, 8, device=DEV)
    bias = torch.tensor([0.3, -0.1, 0.0, 0.1], device=DEV)
    w0, ids0, map0 = base(x, bias)
    w1, ids1, map1 = quantile(x, bias)
    assert torch.equal(ids1, ids0) and torch.equal(w1, w0) and torch.equal(map1, map0)
    hist = quantile.quantile_balancer.required_bias_histogram_EB
    assert hist.is_cuda and int(hist.sum()) == 8 * 4
    # and it matches the oracle's histogram of the same scores
    scores = torch.sigmoid(quantile.gate(x)).cpu()
    _, cutoff = R.select_top_k_plus_one(scores, bias.cpu(), 2)
    want = torch.zeros(4, 1000, dtype=torch.int64)
    R.quantile_observe(want, scores, cutoff, bias.cpu())
    assert int((hist.cpu() - want).abs().sum()) <= 2  # a pair on a bin edge may move with the last ulp of exp


def test_eval_observes_nothing_and_matches_the_base_path_exactly():
    # test_moe_routing.py:211-227
    base, quantile = _routers()
    base.eval(); quantile.eval()
    x = torch.randn(8, 8, device=DEV)
    bias = torch.tensor([0.3, -0.1, 0.0, 0.1], device=DEV)
    _, ids0, _ = base(x, bias)
    _, ids1, _ = quantile(x, bias)
    assert torch.equal(ids1, ids0)
    assert int(quantile.quantile_balancer.required_bias_histogram_EB.sum()) == 0


def test_routing_uses_biased_choice_and_unbiased_weight():
    # test_moe_routing.py:170-182
    _, router = _routers()
    router.eval()
    x = torch.randn(6, 8, device=DEV)
    w, ids, _ = router(x, torch.tensor([10.0, 0.0, 0.0, 0.0], device=DEV))
    assert torch.equal(ids[:, 0], torch.zeros(6, dtype=torch.int64, device=DEV))
    scores = torch.sigmoid(router.gate(x))
    torch.testing.assert_close(w, scores.gather(-1, ids))


def _quantile_moe(E=4, D=4, K=2, bins=10, F=8):
    from torchllmtuner_amd.moe import (GroupedExperts, LocalTokenDispatcher, MoE, QuantileBalancedTopKRouter,
                                       RoutedExperts)

    moe = MoE(E, RoutedExperts(GroupedExperts(D, F, E), LocalTokenDispatcher(E, K)),
              QuantileBalancedTopKRouter(E, D, K, num_bins=bins), load_balance_coeff=None).to(DEV)
    for p in moe.parameters():
        torch.nn.init.normal_(p, std=0.1)
    return moe


def test_the_hook_solves_the_bias_and_drains_the_scratch():
    # test_moe_routing.py:444-475: the worked example through router, hook and optimizer step
    from torchllmtuner_amd.moe import register_moe_balancing_hook

    moe = _quantile_moe()
    moe.train()
    opt = torch.optim.SGD([torch.nn.Parameter(torch.zeros(1))], lr=0.1, foreach=False)
    register_moe_balancing_hook(opt, model_parts=[moe], parallel_dims=None)
    scores = torch.tensor([0.92, 0.68, 0.31, 0.07]).expand(4, -1)
    with torch.no_grad():
        moe.router.gate.weight.copy_(torch.eye(4))
    _, ids, _ = moe.router(torch.logit(scores).to(DEV), moe.expert_bias_E)
    assert torch.equal(ids.cpu(), torch.tensor([[0, 1]] * 4))
    hist = moe.router.quantile_balancer.required_bias_histogram_EB
    assert hist.sum(dim=-1).tolist() == [4, 4, 4, 4]
    moe.tokens_per_expert_E.copy_(torch.tensor([8.0, 8.0, 0.0, 0.0]))
    opt.step()
    torch.testing.assert_close(moe.expert_bias_E.cpu(), torch.tensor([-0.55, -0.15, 0.25, 0.45]))
    assert int(hist.sum()) == 0 and float(moe.tokens_per_expert_E.sum()) == 0.0


def test_block_forward_backward_equals_the_plain_block_with_the_same_bias():
    """A quantile block routes exactly like a sigmoid top-k block holding the same bias, so
    output and gradients agree bit for bit; its histogram sees the unpadded tokens only and
    skips activation-checkpoint replays (test_moe_routing.py:527-581)."""
    from torchllmtuner_amd.moe import (GroupedExperts, LocalTokenDispatcher, MoE, RoutedExperts,
                                       TokenChoiceTopKRouter)
    from torchllmtuner_amd.moe.layer import in_checkpoint_recompute

    E, D, K, F, T = 8, 64, 2, 96, 40
    q = _quantile_moe(E, D, K, bins=32, F=F)
    plain = MoE(E, RoutedExperts(GroupedExperts(D, F, E), LocalTokenDispatcher(E, K)),
                TokenChoiceTopKRouter(E, D, K, score_func="sigmoid"), load_balance_coeff=1e-3).to(DEV)
    plain.load_state_dict(q.state_dict())
    bias = (torch.rand(E) - 0.5) * 0.2
    with torch.no_grad():
        q.expert_bias_E.copy_(bias); plain.expert_bias_E.copy_(bias)
    q.train(); plain.train()
    pad = torch.zeros(T, dtype=torch.bool); pad[[1, 4, 30]] = True
    x = torch.randn(T, D)
    outs = []
    for block in (q, plain):
        xin = x.to(DEV).requires_grad_()
        out = block(xin, padding_mask=pad.to(DEV))
        out.square().sum().backward()
        outs.append((out, xin.grad, block.router.gate.weight.grad, block.routed_experts.inner_experts.w1_EFD.grad))
    for a, b in zip(*outs):
        assert torch.equal(a, b)
    hist = q.router.quantile_balancer.required_bias_histogram_EB
    assert int(hist.sum()) == int((~pad).sum()) * E
    assert torch.equal(q.tokens_per_expert_E, plain.tokens_per_expert_E)
    token = in_checkpoint_recompute.set(True)
    try:
        q(x.to(DEV), padding_mask=pad.to(DEV))
    finally:
        in_checkpoint_recompute.reset(token)
    assert int(hist.sum()) == int((~pad).sum()) * E


def test_the_update_pushes_load_toward_balance():
    # test_moe_routing.py:274-298
    _, router = _routers(num_bins=100)
    router.train()
    with torch.no_grad():
        router.gate.weight.zero_()
        router.gate.weight[0].fill_(4.0)
    x = torch.randn(32, 8, device=DEV).abs()  # expert 0 dominates every token
    bias = torch.zeros(4, device=DEV)
    router(x, bias)
    b = router.quantile_balancer
    nxt = b.estimate_expert_bias(b.required_bias_histogram_EB, bias)
    assert float(nxt[0]) < 0 and float(nxt[1:].max()) > 0 and abs(float(nxt.sum())) < 1e-6
    before = int(router(x, bias)[2][:, 0].sum())
    after = int(router(x, nxt)[2][:, 0].sum())
    assert after <= before
