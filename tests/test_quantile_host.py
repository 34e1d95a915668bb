"""Host-side contracts of quantile-balanced routing (no GPU): constructor validation,
buffers and state dict, policy selection of the balancing hook.  The cases follow
tests/unit_tests/cpu/models/test_moe_routing.py:121-166 and :303-355 of the reference."""

import pytest
import torch

from torchllmtuner_amd import _lib
from torchllmtuner_amd.moe import (
    GroupedExperts,
    LocalTokenDispatcher,
    MoE,
    QuantileBalancedTopKRouter,
    QuantileBalancer,
    RoutedExperts,
    TokenChoiceTopKRouter,
    register_moe_balancing_hook,
    update_quantile_expert_bias,
)

E, D, K = 4, 8, 2


def _moe(router=None, **kw):
    kw.setdefault("load_balance_coeff", None)
    return MoE(E, RoutedExperts(GroupedExperts(D, 8, E), LocalTokenDispatcher(E, K)),
               router or QuantileBalancedTopKRouter(E, D, K), **kw)


def test_a_quantile_moe_carries_a_persistent_bias_buffer_with_no_coeff():
    moe = _moe()
    assert moe.load_balance_coeff is None
    assert torch.equal(moe.expert_bias_E, torch.zeros(E))
    assert "expert_bias_E" in moe.state_dict()


def test_a_coeff_and_a_quantile_router_are_rejected():
    with pytest.raises(ValueError, match="load_balance_coeff must be None"):
        _moe(load_balance_coeff=0.1)


def test_the_histogram_is_int64_scratch_and_not_checkpoint_state():
    router = QuantileBalancedTopKRouter(E, D, K, num_bins=10)
    hist = router.quantile_balancer.required_bias_histogram_EB
    assert hist.dtype == torch.int64 and hist.shape == (E, 10)
    assert "quantile_balancer.required_bias_histogram_EB" not in router.state_dict()
    assert router.score_func == "sigmoid"


def test_top_k_must_leave_a_cutoff_expert():
    with pytest.raises(ValueError, match="top_k"):
        QuantileBalancedTopKRouter(E, D, E)
    for bad in ({"num_experts": 0}, {"top_k": 0}, {"num_bins": 0}, {"num_bins": True}):
        with pytest.raises(ValueError, match="must be positive integer"):
            QuantileBalancer(**({"num_experts": 4, "top_k": 2, "num_bins": 8} | bad))


def test_the_router_refuses_to_route_without_a_bias():
    router = QuantileBalancedTopKRouter(E, D, K)
    with pytest.raises(ValueError, match="requires an expert bias"):
        router(torch.randn(4, D))
    with pytest.raises(ValueError, match="requires an expert bias"):
        router.route(torch.randn(4, D))


class _Model(torch.nn.Module):
    def __init__(self, moes):
        super().__init__()
        self.layers = torch.nn.ModuleList(moes)


def _sgd():
    return torch.optim.SGD([torch.nn.Parameter(torch.zeros(1))], lr=0.1, foreach=False)


def test_a_mixed_model_is_rejected_and_gets_no_hook():
    sign_based = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=0.1)
    opt = _sgd()
    with pytest.raises(ValueError, match="mutually exclusive"):
        register_moe_balancing_hook(opt, model_parts=[_Model([_moe(), sign_based])], parallel_dims=None)
    assert opt._optimizer_step_pre_hooks == {}


def test_inconsistent_coefficients_are_rejected_and_no_balancing_means_no_hook():
    a = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=0.1)
    b = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=None)
    with pytest.raises(ValueError, match="configured consistently"):
        register_moe_balancing_hook(_sgd(), model_parts=[_Model([a, b])], parallel_dims=None)
    opt = _sgd()
    register_moe_balancing_hook(opt, model_parts=[_Model([b])], parallel_dims=None)
    register_moe_balancing_hook(opt, model_parts=[torch.nn.Linear(2, 2)], parallel_dims=None)
    assert opt._optimizer_step_pre_hooks == {}


def test_the_sign_based_hook_steps_the_bias_and_drains_the_counter():
    # test_moe_routing.py:303-331; host tensors only, no kernel involved
    moe = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=0.1)
    opt = _sgd()
    register_moe_balancing_hook(opt, model_parts=[_Model([moe])], parallel_dims=None)
    assert len(opt._optimizer_step_pre_hooks) == 1
    counts = torch.arange(E, dtype=torch.float32)
    moe.tokens_per_expert_E.copy_(counts)
    expected = moe.expert_bias_E + 0.1 * (counts.mean() - counts).sign()
    opt.step()
    torch.testing.assert_close(moe.expert_bias_E, expected)
    assert moe.tokens_per_expert_E.count_nonzero() == 0


def test_reductions_across_processes_are_refused():
    with pytest.raises(NotImplementedError, match="parallel_dims=None"):
        update_quantile_expert_bias([_moe()], parallel_dims=object())


def test_quantile_entry_points_validate_shapes_without_a_gpu():
    lib = _lib.load()
    assert lib.mi355_quantile_observe(None, None, None, None, None, 4, 0, 10, None) != 0
    assert b"quantile_observe" in lib.mi355_moe_last_error()
    assert lib.mi355_quantile_estimate(None, None, None, None, 4, 4, 10, None) != 0  # K must be < E
    assert lib.mi355_router_select_cutoff_fwd(None, None, None, None, None, None, 4, 8, 8, 0, 0, 1.0, None) != 0
    assert b"(K+1)-th" in lib.mi355_moe_last_error()


def test_routing_load_metrics_follow_the_counters():
    # llmtuner/models/common/moe/bias_update.py:100-137
    from torchllmtuner_amd.moe import collect_routing_load_metrics

    a = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=0.1)
    b = _moe(TokenChoiceTopKRouter(E, D, K), load_balance_coeff=0.1)
    model = _Model([a, b])
    assert collect_routing_load_metrics([model], None) == {}          # nothing observed yet
    a.tokens_per_expert_E.copy_(torch.tensor([4.0, 0.0, 2.0, 2.0]))      # mean 2, max 4, one empty
    metrics = collect_routing_load_metrics([model], None)               # b stays inactive
    assert metrics["moe/empty_expert_fraction"] == pytest.approx(0.25)
    assert metrics["moe/max_to_mean_load"] == pytest.approx(2.0)
    assert metrics["moe/load_cv"] == pytest.approx(float(torch.tensor([4.0, 0, 2, 2]).std(unbiased=False)) / 2.0)
    b.tokens_per_expert_E.fill_(3.0)                                    # perfectly even
    metrics = collect_routing_load_metrics([model], None)
    assert metrics["moe/empty_expert_fraction"] == pytest.approx(0.125)
    assert metrics["moe/max_to_mean_load"] == pytest.approx(2.0)
