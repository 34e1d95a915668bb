"""The dispatcher seams of the routed experts (llmtuner/models/common/moe/experts.py:321-343,
llmtuner/parallel/expert_parallel/token_dispatch.py:197-275): a dispatcher that only implements
the reference protocol (``dispatch`` / ``combine`` plus ``num_experts`` / ``top_k``) must work, a
subclass of this package's dispatchers that overrides ``dispatch`` / ``combine`` /
``_permute_tokens`` must be called, and only this package's own, un-overridden dispatchers may be
replaced by the planned / fused kernels.

The CPU tests run the host layer with pure-torch stand-ins for everything that launches a kernel
(router, inner experts, dispatcher), so they pin the control flow; the GPU test runs the
protocol-only dispatcher against the fused path on the device.
"""

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_ref as R
from tests.helpers import build_block, make_params, rel_l2, rel_max
from torchllmtuner_amd import moe
from torchllmtuner_amd.moe.experts import _is_own_dispatcher

T, D, E, K, FF = 24, 16, 4, 2, 32


class ProtocolOnlyDispatcher:
    """Nothing but the reference protocol, in plain torch (token_dispatch.py:146-275)."""

    def __init__(self, num_experts, top_k):
        self.num_experts, self.top_k = num_experts, top_k
        self.accumulate_in_fp32 = False
        self.calls = []

    def set_ep_group(self, *, ep_group=None):
        del ep_group

    def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, num_local_tokens_per_expert_E):
        self.calls.append("dispatch")
        perm = torch.argsort(topk_expert_ids_TK.reshape(-1), stable=True)
        tok = perm // self.top_k
        meta = moe.LocalDispatchMetadata(token_indices_experts_sorted_N=tok,
                                         topk_scores_experts_sorted_N=topk_scores_TK.reshape(-1)[perm])
        return x_TD[tok], num_local_tokens_per_expert_E, meta

    def combine(self, routed_output_RD, metadata, x_TD):
        self.calls.append("combine")
        return R.combine(routed_output_RD, metadata.token_indices_experts_sorted_N,
                         metadata.topk_scores_experts_sorted_N, x_TD, self.accumulate_in_fp32)


class TorchExperts(moe.GroupedExperts):
    """The reference's per-expert loop (experts.py:272-285), so the block runs without a device."""

    def forward(self, x_RD, num_tokens_per_expert_E, *, error_capture=None):
        self.seen_counts = num_tokens_per_expert_E
        out, start = [], 0
        for e, c in enumerate(int(v) for v in num_tokens_per_expert_E.tolist()):
            seg = x_RD[start:start + c]
            out.append(F.linear(F.silu(F.linear(seg, self.w1_EFD[e])) * F.linear(seg, self.w3_EFD[e]), self.w2_EDF[e]))
            start += c
        return torch.cat(out) if out else x_RD.new_zeros(0, self.dim)


class TorchRouter(moe.TokenChoiceTopKRouter):
    """The oracle's routing in place of the device kernels."""

    def forward(self, x_TD, expert_bias_E=None, *, padding_mask_T=None):
        spec = R.RouterSpec(self.num_experts, self.top_k, score_func="softmax", route_norm=True)
        return R.route(R.router_gate(x_TD, self.gate.weight), spec, expert_bias_E)


def _cpu_block(dispatcher):
    p = make_params(E, D, FF, torch.float32, seed=3, std=0.3)
    block = moe.MoE(E, moe.RoutedExperts(TorchExperts(D, FF, E), dispatcher), TorchRouter(E, D, K, route_norm=True),
                    load_balance_coeff=None)
    with torch.no_grad():
        block.router.gate.weight.copy_(p.router_w_ED)
        ie = block.routed_experts.inner_experts
        ie.w1_EFD.copy_(p.w1_EFD); ie.w3_EFD.copy_(p.w3_EFD); ie.w2_EDF.copy_(p.w2_EDF)
    return block, p


def test_protocol_only_dispatcher_runs_the_block_like_the_reference():
    disp = ProtocolOnlyDispatcher(E, K)
    assert not _is_own_dispatcher(disp)
    block, p = _cpu_block(disp)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0))
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    xr = x.clone().requires_grad_()
    ref, aux = R.moe_forward(xr, p, spec)
    ref.backward(torch.ones_like(ref))
    xd = x.clone().requires_grad_()
    out = block(xd)
    out.backward(torch.ones_like(out))
    assert disp.calls == ["dispatch", "combine"]
    # the counts the experts saw are the routing map's column sums (layer.py:278): no plan exists
    assert torch.equal(block.routed_experts.inner_experts.seen_counts, aux["counts_E"])
    assert torch.equal(block.tokens_per_expert_E, aux["counts_E"].float())
    assert rel_max(out, ref) < 1e-6 and rel_max(xd.grad, xr.grad) < 1e-6


def test_protocol_only_dispatcher_without_check_routing_or_plan_attributes():
    """The fallback touches nothing outside the protocol: an object with __slots__ for exactly the
    protocol's attributes survives a forward."""

    class Slotted(ProtocolOnlyDispatcher):
        __slots__ = ()

    disp = Slotted(E, K)
    assert not hasattr(disp, "plan") and not hasattr(disp, "_check_routing")
    block, _ = _cpu_block(disp)
    block(torch.randn(T, D))
    assert disp.calls == ["dispatch", "combine"]


@pytest.mark.parametrize("base", [moe.LocalTokenDispatcher, moe.PaddedTokenDispatcher, moe.LocalShareTokenDispatcher])
@pytest.mark.parametrize("what", ["dispatch", "combine", "_permute_tokens", "plan"])
def test_a_subclass_that_overrides_a_seam_is_not_bypassed(base, what):
    kw = {moe.PaddedTokenDispatcher: {"pad_multiple": 8},
          moe.LocalShareTokenDispatcher: {"local_start": 0, "num_local_experts": 2}}.get(base, {})
    plain = base(E, K, **kw)
    assert _is_own_dispatcher(plain)
    sub = type("Sub", (base,), {})(E, K, **kw)
    assert _is_own_dispatcher(sub), "a subclass that overrides nothing computes the same thing"
    over = type("Over", (base,), {what: lambda self, *a, **k: None})(E, K, **kw)
    assert not _is_own_dispatcher(over)
    patched = base(E, K, **kw)
    setattr(patched, what, lambda *a, **k: None)  # patched on the instance
    assert not _is_own_dispatcher(patched)


def test_overriding_subclass_is_called():
    calls = []

    class Recording(moe.LocalTokenDispatcher):
        def dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, counts_E):
            calls.append(("dispatch", tuple(counts_E.tolist())))
            return ProtocolOnlyDispatcher.dispatch(self, x_TD, topk_scores_TK, topk_expert_ids_TK, counts_E)

        def combine(self, routed_output_RD, metadata, x_TD):
            calls.append(("combine", routed_output_RD.shape[0]))
            return ProtocolOnlyDispatcher.combine(self, routed_output_RD, metadata, x_TD)

    disp = Recording(E, K)
    disp.calls = []
    block, p = _cpu_block(disp)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(1))
    out = block(x)
    ref, aux = R.moe_forward(x, p, R.RouterSpec(E, K, score_func="softmax", route_norm=True))
    assert calls == [("dispatch", tuple(aux["counts_E"].tolist())), ("combine", T * K)]
    assert rel_max(out, ref) < 1e-6


def test_permute_tokens_hook_receives_the_token_of_every_row():
    """An override of _permute_tokens (token_dispatch.py:197-199) is handed the tokens, the token of
    each expert-sorted row and the ids, and its result is what dispatch() returns."""
    from torch._subclasses.fake_tensor import FakeTensorMode

    seen = {}

    class Hooked(moe.LocalTokenDispatcher):
        def _permute_tokens(self, inputs, token_indices, expert_ids):
            seen["args"] = (inputs.shape, token_indices.shape, token_indices.dtype, expert_ids.shape)
            return inputs[token_indices.clamp_min(0)]

    with FakeTensorMode(), torch.device("cuda"):
        disp = Hooked(E, K)
        x = torch.empty(T, D)
        rows, counts, meta = disp.dispatch(x, torch.empty(T, K), torch.empty(T, K, dtype=torch.int64),
                                           torch.empty(E, dtype=torch.int64))
    assert seen["args"] == ((T, D), (T * K,), torch.int64, (T, K))
    assert tuple(rows.shape) == (T * K, D)


def test_plan_memo_key_includes_the_layout():
    from torch._subclasses.fake_tensor import FakeTensorMode

    with FakeTensorMode(), torch.device("cuda"):
        disp = moe.PaddedTokenDispatcher(E, K, pad_multiple=8)
        ids = torch.empty(T, K, dtype=torch.int64)
        plan = disp.plan(ids)
        assert disp.plan(ids) is plan
        disp.pad_multiple = 16  # another layout for the very same ids tensor
        assert disp.plan(ids) is not plan
        share = moe.LocalShareTokenDispatcher(E, K, local_start=0, num_local_experts=2)
        p0 = share.plan(ids)
        share.local_start = 2
        assert share.plan(ids) is not p0
        disp.forget_plan()
        assert disp._last_plan is None


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,Dg,Fg,tol,metric", [(torch.float32, 64, 96, 1e-5, rel_max),
                                                   (torch.bfloat16, 384, 384, 2e-2, rel_l2)])
def test_protocol_fallback_matches_the_fused_path_on_the_device(dtype, Dg, Fg, tol, metric):
    """The same block with this package's dispatcher (planned / fused kernels) and with a
    protocol-only dispatcher in torch ops on the device (dispatch -> GroupedExperts -> combine):
    outputs and every gradient agree within the dtype's bar, and both match the oracle."""
    print(f"protocol fallback {dtype} D={Dg} F={Fg}", flush=True)
    dev = "cuda:0"
    Tg, Eg, Kg = 300, 8, 2
    spec = R.RouterSpec(Eg, Kg, score_func="softmax", route_norm=True)
    p = make_params(Eg, Dg, Fg, dtype, seed=5, std=0.1)
    x = torch.randn(Tg, Dg, generator=torch.Generator().manual_seed(0)).to(dtype)
    gout = torch.randn(Tg, Dg, generator=torch.Generator().manual_seed(1)).to(dtype)

    def run(block):
        xd = x.to(dev).requires_grad_()
        out = block(xd)
        out.backward(gout.to(dev))
        ie = block.routed_experts.inner_experts
        return [out, xd.grad, ie.w1_EFD.grad, ie.w3_EFD.grad, ie.w2_EDF.grad, block.router.gate.weight.grad]

    fused = build_block(p, spec, Dg, Fg, dtype, dev)
    proto = build_block(p, spec, Dg, Fg, dtype, dev)
    disp = ProtocolOnlyDispatcher(Eg, Kg)

    def device_combine(routed_output_RD, metadata, x_TD):  # R.combine allocates on the CPU
        disp.calls.append("combine")
        w = (routed_output_RD.float() * metadata.topk_scores_experts_sorted_N.reshape(-1, 1)).to(routed_output_RD.dtype)
        return torch.zeros_like(x_TD).index_add(0, metadata.token_indices_experts_sorted_N, w)

    disp.combine = device_combine
    proto.routed_experts.token_dispatcher = disp
    a, b = run(fused), run(proto)
    assert disp.calls == ["dispatch", "combine"]
    xr = x.clone().requires_grad_()
    for t in (p.w1_EFD, p.w3_EFD, p.w2_EDF, p.router_w_ED):
        t.requires_grad_()
    ref, _ = R.moe_forward(xr, p, spec)
    ref.backward(gout)
    refs = [ref, xr.grad, p.w1_EFD.grad, p.w3_EFD.grad, p.w2_EDF.grad, p.router_w_ED.grad]
    names = ["out", "dx", "dw1", "dw3", "dw2", "dw_router"]
    for name, u, v, r in zip(names, a, b, refs):
        assert metric(v, u) < tol, f"{name}: protocol path vs fused path {metric(v, u)}"
        if r is not None:
            assert metric(v, r) < tol, f"{name}: protocol path vs oracle {metric(v, r)}"


def test_own_dispatcher_check_gives_a_tracing_compiler_the_eager_answer():
    """RoutedExperts decides between the fused kernels and the protocol calls by looking at the
    dispatcher's four seam methods, instance patches included; a tracing compiler must reach the same
    decision (it cannot read an instance dictionary, and mis-evaluates hasattr on a bound method)."""
    from torchllmtuner_amd import moe
    from torchllmtuner_amd.moe import experts as X

    class Probe(torch.nn.Module):
        def __init__(self, dispatcher):
            super().__init__()
            self.dispatcher = dispatcher

        def forward(self, x):
            return x + 1 if X._is_own_dispatcher(self.dispatcher) else x - 1

    class Other:
        def dispatch(self, *a, **k):
            raise AssertionError

    def free_function(*a, **k):
        raise AssertionError

    cases = {"plain": None, "function on the instance": free_function, "method of another object": Other().dispatch}
    for name, patch in cases.items():
        d = moe.LocalTokenDispatcher(8, 2)
        if patch is not None:
            d.dispatch = patch
        probe = Probe(d)
        want = 1.0 if patch is None else -1.0
        assert probe(torch.zeros(1)).item() == want, name
        torch._dynamo.reset()
        traced = torch.compile(probe, backend="eager", fullgraph=True)
        assert traced(torch.zeros(1)).item() == want, name
