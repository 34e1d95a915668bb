"""The torch.library boundary, checked without a GPU.

The ``mi355_moe`` operators are registered by ``libmi355moe_torch.so``; their fake kernels
(shape / dtype propagation) live in ``torchllmtuner_amd/ops.py``.  Under FakeTensorMode an
operator runs its fake kernel only, so every operator's output contract, and the way the
block's modules call each other, can be exercised here on fake HIP tensors.
"""

import pytest
import torch
from torch._subclasses.fake_tensor import FakeTensorMode

from torchllmtuner_amd import moe, ops

O = torch.ops.mi355_moe
T, D, E, K, F, El = 40, 384, 8, 2, 512, 8
N = T * K
BF, F32, I32, I64 = torch.bfloat16, torch.float32, torch.int32, torch.int64


def _fake(shape, dtype=F32):
    return torch.empty(shape, dtype=dtype, device="cuda")


def _shapes(out):
    out = out if isinstance(out, (tuple, list)) else (out,)
    return [(tuple(t.shape), t.dtype) for t in out]


def _plan_tensors():
    tile_cap = N // ops.TILE_M + El + 1
    return (_fake((El + 1,), I32), _fake((El,), I32), _fake((tile_cap,), I32), _fake((tile_cap,), I32),
            _fake((1,), I32))


def test_every_operator_is_registered_with_a_fake_kernel_and_propagates_shapes():
    expected_ops = {
        "router_gate_fwd", "router_gate_bwd", "router_select_fwd", "router_select_cutoff_fwd", "router_select_bwd",
        "quantile_observe", "quantile_estimate", "rms_norm_fwd", "rms_norm_bwd", "balance_loss_fwd",
        "balance_loss_bwd", "permute_plan", "segments_from_counts", "permute_rows_fwd", "permute_rows_bwd",
        "combine_fwd", "combine_bwd", "combine_row_scale", "combine_scores_bwd", "grouped_swiglu_fwd",
        "grouped_swiglu_bwd", "grouped_linear_fwd", "grouped_linear_bwd", "gather_experts_combine_fwd",
        "gather_experts_combine_bwd", "rows_experts_combine_fwd", "rows_experts_combine_bwd",
    }
    tile_cap = N // ops.TILE_M + El + 1
    small = E + (El + 1) + 2 * El + 2 * tile_cap + 1
    seen = set()
    with FakeTensorMode():
        x, w, logits = _fake((T, D), BF), _fake((E, D)), _fake((T, E))
        ids, wts = _fake((T, K), I64), _fake((T, K))
        w1, w3, w2 = _fake((El, F, D), BF), _fake((El, F, D), BF), _fake((El, D, F), BF)
        ros, sor, tok = _fake((N,), I32), _fake((N,), I32), _fake((N,), I32)
        seg = _plan_tensors()
        rows, rf = _fake((N, D), BF), _fake((N, F), BF)
        cases = {
            "router_gate_fwd": (O.router_gate_fwd(x, w, None), [((T, E), F32)]),
            "router_gate_bwd": (O.router_gate_bwd(logits, x, w, True, False), [((T, D), BF), ((0,), F32)]),
            "router_select_fwd": (O.router_select_fwd(logits, None, K, 1, True, 1.0, 0, 0, 0, True, True),
                                  [((T, K), F32), ((T, K), I64), ((T, E), F32), ((T, E), torch.bool)]),
            "router_select_cutoff_fwd": (O.router_select_cutoff_fwd(logits, _fake((E,)), K, 0, True, 1.0),
                                         [((T, K), F32), ((T, K), I64), ((T, E), F32), ((T,), F32)]),
            "router_select_bwd": (O.router_select_bwd(logits, ids, wts, None, 1, True, 1.0, 0), [((T, E), F32)]),
            "quantile_estimate": (O.quantile_estimate(_fake((E, 100), I64), _fake((E,)), K), [((E,), F32)]),
            "rms_norm_fwd": (O.rms_norm_fwd(_fake((2, T, D), BF), _fake((D,), BF), 1e-6),
                             [((2, T, D), BF), ((2 * T,), F32)]),
            "rms_norm_bwd": (O.rms_norm_bwd(x, x, _fake((D,), BF), _fake((T,)), True, True), [((T, D), BF), ((D,), BF)]),
            "balance_loss_fwd": (O.balance_loss_fwd(logits, _fake((T, E), torch.bool), None), [((1 + E,), F32)]),
            "balance_loss_bwd": (O.balance_loss_bwd(logits, _fake((E,)), None, _fake((1,))), [((T, E), F32)]),
            "permute_plan": (O.permute_plan(ids, E, 0, E, 1), [((small,), I32), ((N,), I32), ((2, N), I32)]),
            "segments_from_counts": (O.segments_from_counts(_fake((El,), I32), N),
                                     [((small - E,), I32)]),
            "permute_rows_fwd": (O.permute_rows_fwd(x, ros, None, seg[4], K, N), [((N, D), BF)]),
            "permute_rows_bwd": (O.permute_rows_bwd(rows, ros, T, K), [((T, D), BF)]),
            "combine_fwd": (O.combine_fwd(rows, wts, ros, None, None, T, K, True), [((T, D), BF)]),
            "combine_bwd": (O.combine_bwd(x, rows, wts, ros, None, None, K), [((N, D), BF), ((T, K), F32)]),
            "combine_row_scale": (O.combine_row_scale(wts, sor, N), [((N,), F32)]),
            "combine_scores_bwd": (O.combine_scores_bwd(_fake((N, 4)), ros, T, K), [((T, K), F32)]),
            "grouped_swiglu_fwd": (O.grouped_swiglu_fwd(rows, None, w1, w3, w2, *seg, N, False),
                                   [((N, D), BF), ((N, F), BF), ((N, F), BF), ((N, F), BF)]),
            "grouped_swiglu_bwd": (O.grouped_swiglu_bwd(rows, rows, None, w1, w3, w2, rf, rf, rf, *seg, True, True, False),
                                   [((N, D), BF), ((El, F, D), BF), ((El, F, D), BF), ((El, D, F), BF)]),
            "grouped_linear_fwd": (O.grouped_linear_fwd(rows, w1, *seg, False), [((N, F), BF)]),
            "grouped_linear_bwd": (O.grouped_linear_bwd(rf, rows, w1, *seg, True, False, False), [((N, D), BF), ((0,), BF)]),
            "rows_experts_combine_fwd": (
                O.rows_experts_combine_fwd(x, wts, w1, w3, w2, ros, None, seg[4], *seg, K, N, True),
                [((T, D), BF), ((N, D), BF), ((N, F), BF), ((N, F), BF), ((N, F), BF), ((N, D), BF)]),
            "rows_experts_combine_bwd": (
                O.rows_experts_combine_bwd(x, rows, wts, w1, w3, w2, rf, rf, rf, rows, ros, None, seg[4], *seg, T, K,
                                           True, True),
                [((T, D), BF), ((El, F, D), BF), ((El, F, D), BF), ((El, D, F), BF), ((T, K), F32)]),
            "gather_experts_combine_fwd": (
                O.gather_experts_combine_fwd(x, wts, w1, w3, w2, tok, sor, ros, *seg, K, N, True, True),
                [((T, D), BF), ((N, F), BF), ((N, F), BF)]),
            "gather_experts_combine_bwd": (
                O.gather_experts_combine_bwd(x, x, wts, w1, w3, w2, rf, rf, tok, sor, ros, *seg, K, True, True),
                [((T, D), BF), ((El, F, D), BF), ((El, F, D), BF), ((El, D, F), BF), ((T, K), F32)]),
        }
        fwd_only = O.gather_experts_combine_fwd(x, wts, w1, w3, w2, tok, sor, ros, *seg, K, N, True, False)
        assert [tuple(t.shape) for t in fwd_only] == [(T, D), (0, F), (0, F)]
        assert O.quantile_observe(_fake((E, 100), I64), logits, _fake((T,)), _fake((E,)), None) is None
        seen.add("quantile_observe")
        for name, (out, want) in cases.items():
            assert _shapes(out) == want, f"{name}: {_shapes(out)} != {want}"
            seen.add(name)
    assert seen == expected_ops


def _fake_block(*, routed_cls=moe.RoutedExperts, dtype=BF):
    router = moe.TokenChoiceTopKRouter(E, D, K, score_func="softmax", route_norm=True)
    torch.set_default_dtype(dtype)
    try:
        experts = moe.GroupedExperts(D, F, E)
    finally:
        torch.set_default_dtype(F32)
    return moe.MoE(E, routed_cls(experts, moe.LocalTokenDispatcher(E, K)), router, load_balance_coeff=None)


def test_block_calls_its_submodules_through_their_hooks():
    """MoE.forward goes through ``self.router(...)`` and ``self.routed_experts(...)`` like
    llmtuner/models/common/moe/layer.py:273-285: forward hooks and pre-hooks on both fire, with
    the reference's argument and result shapes; a hook on the inner experts moves the block off
    the fused kernels so that it fires too."""
    with FakeTensorMode(), torch.device("cuda"):
        block = _fake_block()
        seen = {}
        block.router.register_forward_hook(lambda m, a, out: seen.__setitem__("router", _shapes(out)))
        block.routed_experts.register_forward_pre_hook(lambda m, a: seen.__setitem__("routed_in", _shapes(a)))
        block.routed_experts.register_forward_hook(lambda m, a, out: seen.__setitem__("routed_out", _shapes(out)))
        x = torch.empty(2, T // 2, D, dtype=BF)
        out = block(x)
        assert _shapes(out) == [((2, T // 2, D), BF)]
        assert seen["router"] == [((T, K), F32), ((T, K), I64), ((T, E), torch.bool)]
        assert seen["routed_in"] == [((T, D), BF), ((T, K), F32), ((T, K), I64), ((E,), I32)]
        assert seen["routed_out"] == [((T, D), BF)]
        assert "inner" not in seen
        block.routed_experts.inner_experts.register_forward_hook(
            lambda m, a, out: seen.__setitem__("inner", _shapes(a) + _shapes(out)))
        block(x)
        assert seen["inner"] == [((N, D), BF), ((E,), I32), ((N, D), BF)]


def test_situ_activation_matches_the_explicit_formula_and_validates_its_arguments():
    """The formula and gradient check of tests/unit_tests/cpu/models/test_situ_activation.py:31-45
    and the constructor errors of llmtuner/models/common/activation.py:47-54."""
    for linear_beta in (None, 0.0, 1.7):
        torch.manual_seed(0)
        gate = torch.randn(2, 5, requires_grad=True)
        up = torch.randn(2, 5, requires_grad=True)
        actual = moe.SituGLU(2.0, linear_beta)(gate, up)
        bounded_up = up if not linear_beta else linear_beta * torch.tanh(up / linear_beta)
        expected = 2 * torch.tanh(gate / 2) / (1 + (-gate).exp()) * bounded_up
        torch.testing.assert_close(actual, expected)
        for a, b in zip(torch.autograd.grad(actual.sum(), (gate, up)), torch.autograd.grad(expected.sum(), (gate, up))):
            torch.testing.assert_close(a, b)
    assert moe.SituGLU()(torch.ones(3).bfloat16(), torch.ones(3).bfloat16()).dtype is BF
    for bad in (0.0, -1.0, float("inf"), float("nan")):
        with pytest.raises(ValueError, match="beta must be finite and positive"):
            moe.SituGLU(bad)
    for bad in (-0.5, float("inf")):
        with pytest.raises(ValueError, match="linear_beta must be finite and nonnegative"):
            moe.SituGLU(1.0, bad)
    assert issubclass(moe.SituGLU, moe.ActivationFn) and issubclass(moe.SwiGLU, moe.ActivationFn)
    with pytest.raises(TypeError):
        moe.ActivationFn()  # abstract


def test_a_block_with_another_activation_runs_three_grouped_linear_maps():
    """Only SwiGLU itself is evaluated inside the gate/up kernel: SituGLU, a caller's own module and a
    subclass of SwiGLU (which may compute anything) all run between grouped linear maps, with the
    reference's shapes (experts.py:204-209)."""
    class Mine(moe.SwiGLU):
        def forward(self, gate, up):
            calls.append((tuple(gate.shape), tuple(up.shape)))
            return gate * up

    calls = []
    with FakeTensorMode(), torch.device("cuda"):
        block = _fake_block()
        ie = block.routed_experts.inner_experts
        assert ie.fuses_activation()
        x = torch.empty(T, D, dtype=BF)
        for act in (moe.SituGLU(2.0, 1.0), Mine()):
            ie.activation_fn = act
            assert not ie.fuses_activation()
            assert _shapes(block(x)) == [((T, D), BF)]
            assert _shapes(ie(torch.empty(N, D, dtype=BF), torch.empty(E, dtype=I64))) == [((N, D), BF)]
    assert calls == [((N, F), (N, F))] * 2


def test_a_block_with_a_shared_expert_traces_without_touching_a_stream():
    """Under fake tensors (no device behind them) the shared expert runs in place: the second
    stream is for real device tensors only."""
    with FakeTensorMode(), torch.device("cuda"):
        block = _fake_block()
        torch.set_default_dtype(BF)
        try:
            block.shared_experts = moe.DenseSwiGLU(D, 2 * F)
        finally:
            torch.set_default_dtype(F32)
        assert block.overlap_shared_experts
        x = torch.empty(2, T // 2, D, dtype=BF)
        assert _shapes(block(x)) == [((2, T // 2, D), BF)]
        assert block._start_shared_experts(x.reshape(-1, D)) == (None, None)


def test_a_routed_experts_subclass_that_replaces_forward_is_honoured():
    """The seam the reference names at experts.py:307-311 (DominoRoutedExperts, MC2RoutedExperts,
    KimiRoutedExperts replace ``forward`` wholesale)."""
    calls = []

    class Doubling(moe.RoutedExperts):
        def forward(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
            calls.append((tuple(x_TD.shape), tuple(topk_expert_ids_TK.shape), tuple(num_local_tokens_per_expert_E.shape)))
            return x_TD * 2

    with FakeTensorMode(), torch.device("cuda"):
        block = _fake_block(routed_cls=Doubling)
        assert block.routed_experts.dispatch_observation is None  # only the base class owns one
        out = block(torch.empty(T, D, dtype=BF))
        assert _shapes(out) == [((T, D), BF)]
    assert calls == [((T, D), (T, K), (E,))]


def test_dispatch_observation_wraps_the_fused_path_too():
    entered = []

    class Observer:
        def measure(self, device):
            from contextlib import contextmanager

            @contextmanager
            def cm():
                entered.append(device.type)
                yield

            return cm()

    with FakeTensorMode(), torch.device("cuda"):
        block = _fake_block()
        block.routed_experts.dispatch_observation = moe.DispatchObservation(Observer())
        block(torch.empty(T, D, dtype=BF))                      # fused kernels (bf16, MFMA-sized)
        block32 = _fake_block(dtype=F32)
        block32.routed_experts.dispatch_observation = moe.DispatchObservation(Observer())
        block32(torch.empty(T, D))                              # separate dispatch / experts / combine
    assert entered == ["cuda", "cuda"]


def test_dispatch_metadata_accepts_the_reference_fields():
    """LocalDispatchMetadata(token_indices_experts_sorted_N=..., topk_scores_experts_sorted_N=...)
    as in llmtuner/parallel/expert_parallel/token_dispatch.py:84-89."""
    tok = torch.tensor([0, 1, 1, 2, 0, 2])
    sc = torch.rand(6)
    meta = moe.LocalDispatchMetadata(token_indices_experts_sorted_N=tok, topk_scores_experts_sorted_N=sc)
    assert meta.token_indices_experts_sorted_N is tok and meta.topk_scores_experts_sorted_N is sc
    assert meta.plan is None
    with pytest.raises(TypeError):
        moe.LocalDispatchMetadata(token_indices_experts_sorted_N=tok)


def test_dispatcher_reuses_the_plan_for_the_same_ids_tensor_only():
    with FakeTensorMode(), torch.device("cuda"):
        disp = moe.LocalTokenDispatcher(E, K)
        ids = torch.empty(T, K, dtype=I64)
        plan = disp.plan(ids)
        assert disp.plan(ids) is plan
        assert disp.plan(ids.clone()) is not plan
        ids2 = torch.empty(T, K, dtype=I64)
        p2 = disp.plan(ids2)
        ids2.add_(1)  # changed in place: a new plan
        assert disp.plan(ids2) is not p2


def test_exit_hook_is_idle_without_a_gpu():
    """The package's exit hook (it lets the autograd engine's thread take the GIL once more before the
    interpreter finalises) costs nothing in a process that never initialised the GPU."""
    import atexit
    import time

    from torchllmtuner_amd import ops

    assert callable(ops._let_autograd_threads_finish)
    atexit.unregister(ops._let_autograd_threads_finish)  # (what import registered; put back below)
    atexit.register(ops._let_autograd_threads_finish)
    if not torch.cuda.is_initialized():
        t0 = time.perf_counter()
        ops._let_autograd_threads_finish()
        assert time.perf_counter() - t0 < 0.02
