"""HF-style packed experts -> native block, and the expert key mapping.

Expectations restate the reference's own checks: ``gate_up_proj[:, :F]`` is ``w1_EFD`` and
``[:, F:]`` is ``w3_EFD`` (tests/unit_tests/cpu/parallel/test_ep_model_replacement.py:395-417),
fp32 router and fp32 state buffers under bf16 experts (:1172-1206), key rules of
llmtuner/models/qwen/qwen3/state.py:14-103, and per-expert HF math
``down(act(gate(x)) * up(x))`` (:420-448).
"""

import pytest
import torch

from torchllmtuner_amd import moe

E, D, F, K = 6, 16, 12, 2


def _packed(dtype=torch.bfloat16, seed=0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(E, D, generator=g) * 0.1,
            (torch.randn(E, 2 * F, D, generator=g) * 0.1).to(dtype),
            (torch.randn(E, D, F, generator=g) * 0.1).to(dtype))


def test_packed_tensors_land_in_the_native_parameters():
    rw, gu, dn = _packed()
    bias = torch.linspace(-1, 1, E)
    block = moe.moe_from_packed_experts(rw, gu, dn, top_k=K, score_func="sigmoid", route_norm=True,
                                        e_score_correction_bias=bias)
    sd = block.state_dict()
    assert sorted(sd) == ["expert_bias_E", "routed_experts.inner_experts.w1_EFD",
                          "routed_experts.inner_experts.w2_EDF", "routed_experts.inner_experts.w3_EFD",
                          "router.gate.weight"]
    assert torch.equal(sd["routed_experts.inner_experts.w1_EFD"], gu[:, :F])
    assert torch.equal(sd["routed_experts.inner_experts.w3_EFD"], gu[:, F:])
    assert torch.equal(sd["routed_experts.inner_experts.w2_EDF"], dn)
    assert torch.equal(sd["router.gate.weight"], rw) and sd["router.gate.weight"].dtype == torch.float32
    assert torch.equal(sd["expert_bias_E"], bias) and sd["expert_bias_E"].dtype == torch.float32
    assert block.tokens_per_expert_E.dtype == torch.float32 and block.load_balance_coeff == 1e-3
    assert block.training and block.router.top_k == K and block.router.aux_loss is None
    # no bias buffer in the source model: no bias state in the block
    plain = moe.moe_from_packed_experts(rw, gu, dn, top_k=K)
    assert plain.expert_bias_E is None and "expert_bias_E" not in plain.state_dict()


def test_options_select_dispatcher_aux_loss_and_local_share():
    rw, gu, dn = _packed()
    padded = moe.moe_from_packed_experts(rw, gu, dn, top_k=K, token_dispatcher="torchao", torchao_pad_multiple=32,
                                         router_aux_loss_coef=0.01, fixed_router=True, training=False)
    disp = padded.routed_experts.token_dispatcher
    assert isinstance(disp, moe.PaddedTokenDispatcher) and disp.pad_multiple == 32
    assert isinstance(padded.router.aux_loss, moe.MicrobatchWiseLoadBalanceLoss) and padded.router.aux_loss.coeff == 0.01
    assert padded.router.fixed_router and not padded.training
    share = moe.moe_from_packed_experts(rw, gu, dn, top_k=K, local_experts=(2, 5))
    assert isinstance(share.routed_experts.token_dispatcher, moe.LocalShareTokenDispatcher)
    assert torch.equal(share.routed_experts.inner_experts.w2_EDF, dn[2:5])
    assert share.router.gate.weight.shape == (E, D)
    with pytest.raises(ValueError, match="more than one process"):
        moe.moe_from_packed_experts(rw, gu, dn, top_k=K, token_dispatcher="alltoall")
    with pytest.raises(ValueError, match="do not agree"):
        moe.moe_from_packed_experts(rw, gu[:, :-1], dn, top_k=K)
    frozen = moe.moe_from_packed_experts(rw, gu.requires_grad_(False), dn.requires_grad_(True), top_k=K)
    ie = frozen.routed_experts.inner_experts
    assert not ie.w1_EFD.requires_grad and not ie.w3_EFD.requires_grad and ie.w2_EDF.requires_grad


def test_expert_key_mapping_round_trip():
    pre = "model.layers.3.mlp."
    assert moe.native_ep_expert_key(pre + "experts.7.up_proj.weight") == pre + "routed_experts.inner_experts.w3_EFD"
    assert moe.native_ep_expert_key(pre + "experts.0.gate_proj.weight") == pre + "routed_experts.inner_experts.w1_EFD"
    assert moe.native_ep_expert_key(pre + "experts.1.down_proj.weight") == pre + "routed_experts.inner_experts.w2_EDF"
    assert moe.native_ep_expert_key(pre + "gate.weight") == pre + "gate.weight"
    g = torch.Generator().manual_seed(1)
    hf = {pre + "gate.weight": torch.randn(E, D, generator=g)}
    for e in range(E):
        hf[pre + f"experts.{e}.gate_proj.weight"] = torch.randn(F, D, generator=g)
        hf[pre + f"experts.{e}.up_proj.weight"] = torch.randn(F, D, generator=g)
        hf[pre + f"experts.{e}.down_proj.weight"] = torch.randn(D, F, generator=g)
    native = moe.hf_expert_state_to_native(hf)
    assert sorted(native) == sorted([pre + "gate.weight", pre + "routed_experts.inner_experts.w1_EFD",
                                     pre + "routed_experts.inner_experts.w3_EFD",
                                     pre + "routed_experts.inner_experts.w2_EDF"])
    assert native[pre + "routed_experts.inner_experts.w1_EFD"].shape == (E, F, D)
    assert torch.equal(native[pre + "routed_experts.inner_experts.w2_EDF"][4], hf[pre + "experts.4.down_proj.weight"])
    back = moe.native_expert_state_to_hf(native, num_experts=E)
    assert sorted(back) == sorted(hf) and all(torch.equal(back[k], hf[k]) for k in hf)
    with pytest.raises(ValueError, match="full expert stack"):
        moe.native_expert_state_to_hf({pre + "routed_experts.inner_experts.w1_EFD": torch.zeros(E - 1, F, D)},
                                      num_experts=E)
    del hf[pre + "experts.2.up_proj.weight"]
    with pytest.raises(ValueError, match="incomplete"):
        moe.hf_expert_state_to_native(hf)


@pytest.mark.gpu
def test_converted_block_computes_the_hf_expert_math():
    """out[t] = sum_k w_k * down_e(silu(gate_e x) * up_e x) with gate/up the two halves of
    gate_up_proj, on tensors placed on the device before conversion."""
    dev = "cuda:0"
    Dg, Fg, Eg, Kg, T = 384, 384, 8, 2, 200
    g = torch.Generator().manual_seed(2)
    rw = torch.randn(Eg, Dg, generator=g) * 0.1
    gu = (torch.randn(Eg, 2 * Fg, Dg, generator=g) * 0.05).bfloat16()
    dn = (torch.randn(Eg, Dg, Fg, generator=g) * 0.05).bfloat16()
    x = torch.randn(T, Dg, generator=g).bfloat16()
    block = moe.moe_from_packed_experts(rw.to(dev), gu.to(dev), dn.to(dev), top_k=Kg, score_func="softmax",
                                        route_norm=True, training=False)
    out = block(x.to(dev)).float().cpu()
    with torch.no_grad():
        w, ids = block.router.route(x.to(dev))
    w, ids = w.cpu(), ids.cpu()
    bf = lambda v: v.bfloat16().float()
    ref = torch.zeros(T, Dg)
    for t in range(T):
        for k in range(Kg):
            e = int(ids[t, k])
            gate, up = bf(gu[e, :Fg].float() @ x[t].float()), bf(gu[e, Fg:].float() @ x[t].float())
            ref[t] += float(w[t, k]) * bf(dn[e].float() @ bf(bf(torch.nn.functional.silu(gate)) * up))
    assert (out - ref).norm() / ref.norm() < 2e-2


# ---- convert_block: the reference's own entry, fed with objects that merely LOOK like its bindings
class _Gate(torch.nn.Module):
    """An HF-style router gate: ``weight (E, D)`` and the aux-loss-free correction bias."""

    def __init__(self, weight, bias=None):
        super().__init__()
        self.weight = torch.nn.Parameter(weight.clone())
        if bias is not None:
            self.register_buffer("e_score_correction_bias", bias.clone())


def _bindings(dtype=torch.bfloat16, bias=None, shared=None, **routing):
    """Plain stand-ins with the fields of MoERoutingBinding / PackedExpertBinding /
    PackedExpertViews (llmtuner/parallel/expert_parallel/bindings.py:36-170); none of the
    reference's classes is imported."""
    from collections import namedtuple
    from types import SimpleNamespace

    rw, gu, dn = _packed(dtype)
    fields = dict(top_k=K, score_func="sigmoid", route_norm=True, route_scale=2.5, num_expert_groups=None,
                  num_limited_groups=None)
    fields.update(routing)
    routing_binding = SimpleNamespace(source=None, router=_Gate(rw, bias), shared=shared, shared_gate=None, **fields)
    views = namedtuple("PackedExpertViews", "gate_EFD up_EFD down_EDF num_experts")(gu[:, :F], gu[:, F:], dn, E)
    binding = SimpleNamespace(gate_up=torch.nn.Parameter(gu.clone()), down=torch.nn.Parameter(dn.clone()),
                              shape=tuple(gu.shape))
    return routing_binding, views, binding, (rw, gu, dn)


def test_convert_block_accepts_the_reference_binding_objects_by_their_fields():
    bias = torch.linspace(-1, 1, E)
    shared = moe.DenseSwiGLU(D, F)
    routing, views, binding, (rw, gu, dn) = _bindings(bias=bias, shared=shared)
    source = torch.nn.Module().eval()  # the HF block being replaced: supplies the mode
    for packed in (views, binding):
        block = moe.convert_block(source, routing=routing, packed_experts=packed, ep_group=None,
                                  aux_loss_coeff=0.01, load_balance_coeff=1e-3, quantile_balancing=False,
                                  token_dispatcher="alltoall", torchao_pad_multiple=16)
        ie = block.routed_experts.inner_experts
        assert torch.equal(ie.w1_EFD, gu[:, :F]) and torch.equal(ie.w3_EFD, gu[:, F:]) and torch.equal(ie.w2_EDF, dn)
        assert ie.w1_EFD.dtype == torch.bfloat16
        assert torch.equal(block.router.gate.weight, rw) and block.router.gate.weight.dtype == torch.float32
        assert torch.equal(block.expert_bias_E, bias) and block.expert_bias_E.dtype == torch.float32
        assert block.shared_experts is shared and not block.training
        r = block.router
        assert (r.top_k, r.score_func, r.route_norm, r.route_scale) == (K, "sigmoid", True, 2.5)
        assert isinstance(r.aux_loss, moe.MicrobatchWiseLoadBalanceLoss) and r.aux_loss.coeff == 0.01
        assert isinstance(block.routed_experts.token_dispatcher, moe.LocalTokenDispatcher)
    # a binding that can validate itself is asked to
    calls = []
    routing.validate = lambda blk: calls.append(blk)
    padded = moe.convert_block(source, routing=routing, packed_experts=views, token_dispatcher="torchao",
                               torchao_pad_multiple=32, load_balance_coeff=None)
    assert calls == [source] and padded.expert_bias_E is None
    assert padded.routed_experts.token_dispatcher.pad_multiple == 32


def test_convert_block_quantile_balancing_and_what_one_gpu_refuses():
    routing, views, _, _ = _bindings()
    q = moe.convert_block(None, routing=routing, packed_experts=views, quantile_balancing=True)
    assert isinstance(q.router, moe.QuantileBalancedTopKRouter) and q.load_balance_coeff is None
    assert q.expert_bias_E is not None and q.training
    soft, views2, _, _ = _bindings(score_func="softmax")
    with pytest.raises(ValueError, match="sigmoid"):
        moe.convert_block(None, routing=soft, packed_experts=views2, quantile_balancing=True)
    for kw, needle in ((dict(ep_group=object()), "one GPU"), (dict(tp_enabled=True), "tensor parallelism"),
                       (dict(token_dispatcher="domino"), "peers")):
        with pytest.raises(NotImplementedError, match=needle):
            moe.convert_block(None, routing=routing, packed_experts=views, **kw)
    with pytest.raises(TypeError, match="packed_experts"):
        moe.convert_block(None, routing=routing, packed_experts=object())
