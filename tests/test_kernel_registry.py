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
