"""The swap the reference performs, end to end, against the block it swaps out.

The reference replaces HuggingFace's ``Qwen3MoeSparseMoeBlock`` by its native block and
copies the weights over (llmtuner/parallel/expert_parallel/block_conversion.py:160-300);
the swap is only legitimate if both blocks compute the same function.  Here the
HuggingFace block (installed ``transformers``, random weights, run in fp32 on the CPU) is
that function's independent statement: the device block built from its packed tensors by
``moe_from_packed_experts`` must reproduce its output and every gradient.
"""

import pytest
import torch

from tests.helpers import rel_l2, rel_max

pytestmark = pytest.mark.gpu
DEV = "cuda:0"

try:
    from transformers.models.qwen3_moe.configuration_qwen3_moe import Qwen3MoeConfig
    from transformers.models.qwen3_moe.modeling_qwen3_moe import Qwen3MoeSparseMoeBlock
except Exception:  # pragma: no cover - transformers absent or too old
    Qwen3MoeSparseMoeBlock = None


def _hf_block(D, F, E, K, seed):
    cfg = Qwen3MoeConfig(hidden_size=D, moe_intermediate_size=F, num_experts=E, num_experts_per_tok=K,
                         norm_topk_prob=True, hidden_act="silu")
    block = Qwen3MoeSparseMoeBlock(cfg).float()
    if not hasattr(block.experts, "gate_up_proj"):
        pytest.skip("this transformers version does not pack the expert weights")
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        # bf16-representable values, so that the bf16 device block starts from the same numbers
        block.gate.weight.copy_((torch.randn(E, D, generator=g) * 0.05).bfloat16().float())
        block.experts.gate_up_proj.copy_((torch.randn(E, 2 * F, D, generator=g) * 0.05).bfloat16().float())
        block.experts.down_proj.copy_((torch.randn(E, D, F, generator=g) * 0.05).bfloat16().float())
    return block


@pytest.mark.skipif(Qwen3MoeSparseMoeBlock is None, reason="transformers with Qwen3-MoE is not installed")
@pytest.mark.parametrize("dtype,D,F,E,K,T", [
    (torch.float32, 64, 96, 8, 2, 300),       # generic fp32 kernels
    (torch.bfloat16, 384, 384, 16, 4, 512),   # bf16 MFMA kernels, token gather fused
])
def test_native_block_reproduces_the_huggingface_block(dtype, D, F, E, K, T):
    print(f"hf swap {dtype} D={D} F={F} E={E} K={K} T={T}", flush=True)
    from torchllmtuner_amd.moe import moe_from_packed_experts

    hf = _hf_block(D, F, E, K, seed=3)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(2, T // 2, D, generator=g).bfloat16().float()
    gout = torch.randn(2, T // 2, D, generator=g).bfloat16().float()

    xr = x.clone().requires_grad_()
    ref = hf(xr)
    ref.backward(gout)

    native = moe_from_packed_experts(
        hf.gate.weight.detach().to(DEV),                       # router stays fp32
        hf.experts.gate_up_proj.detach().to(DEV, dtype),
        hf.experts.down_proj.detach().to(DEV, dtype),
        top_k=K, score_func="softmax", route_norm=True,
    )
    for prm in native.parameters():
        prm.requires_grad_(True)
    xd = x.to(DEV, dtype).requires_grad_()
    out = native(xd)
    out.backward(gout.to(DEV, dtype))

    ie = native.routed_experts.inner_experts
    dgu = hf.experts.gate_up_proj.grad
    pairs = {
        "out": (out, ref), "dx": (xd.grad, xr.grad),
        "router": (native.router.gate.weight.grad, hf.gate.weight.grad),
        "w1": (ie.w1_EFD.grad, dgu[:, :F]), "w3": (ie.w3_EFD.grad, dgu[:, F:]),
        "w2": (ie.w2_EDF.grad, hf.experts.down_proj.grad),
    }
    if dtype == torch.float32:
        for name, (got, want) in pairs.items():
            assert rel_max(got, want) < 1e-5, f"{name}: {rel_max(got, want)}"
    else:
        for name, (got, want) in pairs.items():
            assert rel_l2(got, want) < 2e-2, f"{name}: {rel_l2(got, want)}"
