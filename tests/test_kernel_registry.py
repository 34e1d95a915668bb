"""The kernel-registry seam: registry semantics on the CPU, the permute operator on the GPU.

The cases restate the reference's own contract tests for this interface
(tests/unit_tests/cpu/kernel/test_kernel_contracts.py:16-71 registry behaviour,
:114-140 the permute operator, tests/integration_tests/kernel_equivalence.py:117-152
the device-equivalence inputs).
"""

import logging

import pytest
import torch

from torchllmtuner_amd import kernel_registry as registry
from torchllmtuner_amd.kernel_registry import (
    dispatch_kernel,
    get_kernel,
    moe_token_permute,
    register_kernel,
)


@pytest.fixture
def isolated_registry(monkeypatch):
    monkeypatch.setattr(
        registry, "_KERNEL_REGISTRY",
        {name: dict(backends) for name, backends in registry._KERNEL_REGISTRY.items()})
    monkeypatch.setattr(registry, "_warned_fallbacks", set())


def test_lookup_errors_and_explicit_fallback_warns_once(isolated_registry, caplog):
    with pytest.raises(KeyError, match="not registered"):
        get_kernel("missing_kernel", "cpu")
    with pytest.raises(KeyError, match="not available"):
        get_kernel("moe_token_permute", "unknown")
    # no torch-math backend ships, so the fallback has nothing to fall back to
    with pytest.raises(KeyError, match="not available"):
        get_kernel("moe_token_permute", "unknown", fallback_to_cpu=True)

    def host_kernel():
        return "host"

    register_kernel("custom", "cpu")(host_kernel)
    with caplog.at_level(logging.WARNING):
        for _ in range(2):
            assert get_kernel("custom", "unknown", fallback_to_cpu=True) is host_kernel
    assert len(caplog.records) == 1


@pytest.mark.parametrize("name,device", [("", "cpu"), ("a", ""), (None, "cpu")])
def test_registry_rejects_invalid_identifiers(name, device):
    with pytest.raises(ValueError, match="must not be empty"):
        register_kernel(name, device)


def test_registry_rejects_noncallables_and_accepts_idempotent_registration(isolated_registry):
    with pytest.raises(TypeError, match="callable"):
        register_kernel("custom", "cpu")(None)

    def kernel():
        return 42

    for _ in range(2):
        assert register_kernel("custom", "cpu")(kernel) is kernel
    assert dispatch_kernel("custom", device_type="cpu") == 42
    with pytest.raises(ValueError, match="already registered"):
        register_kernel("custom", "cpu")(lambda: 0)


def test_dispatch_follows_the_tensor_device(isolated_registry):
    seen = []
    register_kernel("probe", "cpu")(lambda *a, **k: seen.append("cpu"))
    register_kernel("probe", "cuda")(lambda *a, **k: seen.append("cuda"))
    dispatch_kernel("probe", 3, values=torch.ones(2))
    dispatch_kernel("probe", torch.ones(2), device_type="cuda")
    dispatch_kernel("probe")  # tensor-free: the package's default device type
    assert seen == ["cpu", "cuda", "cuda"]


def test_permute_operator_is_registered_for_the_gpu_only():
    assert get_kernel("moe_token_permute", "cuda") is registry.moe_token_permute_mi355
    assert set(registry._KERNEL_REGISTRY["moe_token_permute"]) == {"cuda"}
    with pytest.raises(KeyError, match="not available"):
        moe_token_permute(torch.ones(2, 4), torch.zeros(2, 1, dtype=torch.int64))
    with pytest.raises(NotImplementedError, match="only implementation"):
        moe_token_permute(torch.ones(2, 4), torch.zeros(2, 1, dtype=torch.int64), use_eager=True)


@pytest.mark.parametrize(
    "shape,dtype", [((2,), torch.int64), ((2, 0), torch.int64), ((2, 1), torch.float32)])
def test_permute_backend_rejects_invalid_expert_ids(shape, dtype):
    with pytest.raises(ValueError):
        registry.moe_token_permute_mi355(torch.ones(2, 4), torch.zeros(shape, dtype=dtype))
    with pytest.raises(ValueError, match="token counts"):
        registry.moe_token_permute_mi355(torch.ones(3, 4), torch.zeros(2, 1, dtype=torch.int64))


# ------------------------------------------------------------------ GPU
DEV = "cuda:0"


@pytest.mark.gpu
@pytest.mark.parametrize("ids_dtype", [torch.int32, torch.int64])
def test_stable_permutation_and_duplicate_assignment_backward(ids_dtype):
    x = torch.arange(12, dtype=torch.float32, device=DEV).reshape(3, 4).requires_grad_()
    experts = torch.tensor([[2, 0], [0, 0], [2, 1]], dtype=ids_dtype, device=DEV)
    rows = [0, 1, 1, 2, 0, 2]  # sorted by (expert, flattened assignment order)
    actual = moe_token_permute(x, experts)
    assert torch.equal(actual, x.detach()[rows])
    weights = torch.arange(1, 25, dtype=x.dtype, device=DEV).reshape(6, 4)
    (actual * weights).sum().backward()
    expected = torch.stack([weights[0] + weights[4], weights[1] + weights[2], weights[3] + weights[5]])
    assert torch.equal(x.grad, expected)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_permute_matches_stable_argsort(dtype):
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 64, generator=g).to(dtype)
    ids = torch.tensor([[2, 0], [1, 2], [0, 1], [2, 0], [1, 1], [0, 2]], dtype=torch.int32)
    want = x[torch.argsort(ids.reshape(-1), stable=True) // 2]
    got = moe_token_permute(x.to(DEV), ids.to(DEV))
    assert torch.equal(got.cpu(), want)
    # a larger ragged case, number of experts supplied (no host read-back)
    T, K, E, D = 777, 6, 40, 200
    x = torch.randn(T, D, generator=g).to(dtype)
    ids = torch.randint(0, E, (T, K), generator=g)
    ids[ids == 7] = 8  # an expert nobody picks
    want = x[torch.argsort(ids.reshape(-1), stable=True) // K]
    got = moe_token_permute(x.to(DEV), ids.to(DEV), num_experts=E)
    assert torch.equal(got.cpu(), want)


@pytest.mark.gpu
def test_empty_permutation_retains_autograd_and_negative_ids_raise():
    x = torch.empty(0, 4, device=DEV, requires_grad=True)
    result = moe_token_permute(x, torch.empty(0, 2, dtype=torch.int64, device=DEV))
    assert result.shape == (0, 4) and result.requires_grad
    with pytest.raises(ValueError, match="non-negative"):
        moe_token_permute(torch.ones(2, 4, device=DEV), torch.tensor([[0], [-1]], device=DEV))


# ------------------------------------------------------------------ rms_norm
def test_rms_norm_is_registered_for_the_gpu_only_and_validates_metadata():
    from torchllmtuner_amd.kernel_registry import rms_norm, rms_norm_mi355

    assert get_kernel("rms_norm", "cuda") is rms_norm_mi355
    assert set(registry._KERNEL_REGISTRY["rms_norm"]) == {"cuda"}
    with pytest.raises(KeyError, match="not available"):
        rms_norm(torch.ones(2, 4), torch.ones(4), 1e-6)
    with pytest.raises(NotImplementedError, match="only implementation"):
        rms_norm(torch.ones(2, 4), torch.ones(4), 1e-6, use_eager=True)
    # tests/unit_tests/cpu/kernel/test_kernel_contracts.py:108-111 and validation.py:110-120
    for epsilon in (-1.0, float("nan"), float("inf")):
        with pytest.raises(ValueError, match="epsilon"):
            rms_norm_mi355(torch.ones(2, 4), torch.ones(4), epsilon)
    with pytest.raises(ValueError, match="1-D weight"):
        rms_norm_mi355(torch.ones(2, 4), torch.ones(1, 4), 1e-6)
    with pytest.raises(ValueError, match="must match"):
        rms_norm_mi355(torch.ones(2, 4), torch.ones(5), 1e-6)
    with pytest.raises(RuntimeError, match="HIP device"):
        rms_norm_mi355(torch.ones(2, 4), torch.ones(4), 1e-6)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", [(2, 3, 8), (300, 2048), (5, 100), (7, 1), (7, 2), (0, 64), (4, 2, 7168), (33, 4100)])
def test_rms_norm_matches_the_oracle_forward_and_backward(dtype, shape):
    from oracle import moe_ref as R
    from tests.helpers import rel_l2, rel_max
    from torchllmtuner_amd.kernel_registry import rms_norm

    print(f"rms_norm {dtype} {shape}", flush=True)
    g = torch.Generator().manual_seed(sum(shape))
    x = (torch.randn(*shape, generator=g) * 2).to(dtype)
    w = (1 + 0.3 * torch.randn(shape[-1], generator=g)).to(dtype)
    dy = torch.randn(*shape, generator=g).to(dtype)
    xr, wr = x.clone().requires_grad_(), w.clone().requires_grad_()
    want = R.rms_norm(xr, wr, 1e-5)
    want.backward(dy)
    xd, wd = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    got = rms_norm(xd, wd, 1e-5)
    got.backward(dy.to(DEV))
    assert got.shape == want.shape and got.dtype == dtype
    if x.numel() == 0:
        assert xd.grad.shape == x.shape and float(wd.grad.abs().sum()) == 0.0
        return
    metric, tol = (rel_max, 1e-5) if dtype == torch.float32 else (rel_l2, 2e-2)
    assert metric(got, want) < tol
    assert metric(wd.grad, wr.grad) < tol
    if shape[-1] == 1:
        # dx of a one-element row is the difference of two equal terms (eps apart): compare it
        # on the scale of those terms, which is the scale both sides round at
        scale = float((dy.float() * w.float()).abs().max() / x.float().abs().min())
        assert float((xd.grad.cpu().float() - xr.grad.float()).abs().max()) < 1e-5 * max(scale, 1.0)
    else:
        assert metric(xd.grad, xr.grad) < tol
    if dtype == torch.bfloat16:
        # one rounding at the end: at most one bf16 ulp from the library routine
        ulp = want.detach().float().abs() * 2.0 ** -7 + 1e-30
        assert bool(((got.detach().cpu().float() - want.detach().float()).abs() <= ulp).all())


@pytest.mark.gpu
def test_rms_norm_formula_in_front_of_the_block():
    """The decoder layer's `mlp(norm(hidden))` (models/qwen/qwen3/model.py:452) with both halves
    on the device kernels: gradients flow through the block into the norm."""
    import torchllmtuner_amd as amd
    from torchllmtuner_amd.kernel_registry import rms_norm

    E, K, D, Fd = 8, 2, 64, 96
    block = amd.MoE(E, amd.RoutedExperts(amd.GroupedExperts(D, Fd, E), amd.LocalTokenDispatcher(E, K)),
                    amd.TokenChoiceTopKRouter(E, D, K, score_func="softmax", route_norm=True),
                    load_balance_coeff=None).to(DEV)
    for p in block.parameters():
        torch.nn.init.normal_(p, std=0.1)
    hidden = torch.randn(2, 16, D, device=DEV, requires_grad=True)
    weight = torch.ones(D, device=DEV, requires_grad=True)
    out = hidden + block(rms_norm(hidden, weight, 1e-6))
    out.square().sum().backward()
    assert hidden.grad.shape == hidden.shape and torch.isfinite(hidden.grad).all()
    assert weight.grad.shape == (D,) and float(weight.grad.abs().sum()) > 0
