"""GPU parity of the whole MoE block (module API) against the CPU oracle.

Configurations follow the benchmark's list: C1 tiny fp32 fwd+bwd, the Qwen3-30B-A3B
shape in bf16 at a reduced token count (full weights are compared on a sample of
experts), the skewed 128-row padded variant, and the DeepSeek-V3-shaped local-share
block with a shared expert.
"""

import pytest
import torch

from oracle import moe_ref as R
from tests.helpers import build_block, make_params, note, rel_l2, rel_max, stable_tokens
from torchllmtuner_amd.workloads import zipf_logit_bias

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _run_pair(p, spec, x, gout, dtype, D, F, **kw):
    """Oracle fwd+bwd on CPU and device block fwd+bwd; returns both sides' tensors."""
    oracle_kw = {}
    if kw.get("dispatcher") == "padded":
        oracle_kw["pad_multiple"] = kw["pad_multiple"]
    if kw.get("dispatcher") == "share":
        oracle_kw["local_experts"] = kw["local"]
    leaves = {k: getattr(p, k).clone().requires_grad_() for k in
              ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF", "shared_gate_FD", "shared_up_FD", "shared_down_DF")
              if getattr(p, k) is not None}
    pr = R.MoEParams(expert_bias_E=p.expert_bias_E, router_logit_bias_E=p.router_logit_bias_E, **leaves)
    xr = x.clone().requires_grad_()
    if kw.get("activation") is not None:  # the module itself is the oracle's (gate, up) function: plain torch on the CPU
        oracle_kw["activation"] = kw["activation"]
    ref, aux = R.moe_forward(xr, pr, spec, **oracle_kw)
    ref.backward(gout)
    block = build_block(p, spec, D, F, dtype, DEV, load_balance_coeff=1e-3 if p.expert_bias_E is not None else None, **kw)
    block.train()
    xd = x.to(DEV).requires_grad_()
    out = block(xd)
    out.backward(gout.to(DEV))
    ie = block.routed_experts.inner_experts
    got = {"out": out, "dx": xd.grad, "router_w_ED": block.router.gate.weight.grad,
           "w1_EFD": ie.w1_EFD.grad, "w3_EFD": ie.w3_EFD.grad, "w2_EDF": ie.w2_EDF.grad}
    want = {"out": ref, "dx": xr.grad, **{k: v.grad for k, v in leaves.items()}}
    if block.shared_experts is not None:
        got["shared_gate_FD"] = block.shared_experts.gate_proj.weight.grad
        got["shared_up_FD"] = block.shared_experts.up_proj.weight.grad
        got["shared_down_DF"] = block.shared_experts.down_proj.weight.grad
    return got, want, aux, block


def test_c1_tiny_fp32_forward_backward():
    """T=512 (2x256), D=256, E=8, F=512, softmax top-2 with norm, everything fp32."""
    print("block C1", flush=True)
    T, D, E, K, F = 512, 256, 8, 2, 512
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.float32, seed=0)
    x = torch.randn(2, 256, D, generator=torch.Generator().manual_seed(0))
    gout = torch.randn(2, 256, D, generator=torch.Generator().manual_seed(1))
    got, want, aux, block = _run_pair(p, spec, x, gout, torch.float32, D, F)
    ok = stable_tokens(aux["logits"], spec)
    assert ok.all(), "seeded C1 inputs contain a near-tie token"
    # routing bit-exact
    scores, ids = block.router.route(x.reshape(-1, D).to(DEV))
    assert torch.equal(ids.cpu(), aux["ids_TK"])
    assert torch.equal(block.tokens_per_expert_E.cpu().long(), aux["counts_E"])
    assert got["out"].shape == (2, 256, D)
    for k in want:
        assert rel_max(got[k], want[k]) < 1e-5, f"{k}: {rel_max(got[k], want[k])}"


def _check_routing(block, x_dev, aux, spec, expert_bias=None, label=""):
    """Device routing against the oracle's: every token whose ids differ must be a few-ulp near
    tie of the oracle's own scores (the two sides' logits come from differently ordered fp32
    sums), the number of such tokens is printed and bounded, and the block's counters equal the
    bincount of the DEVICE's ids always -- and the oracle's counts whenever no token differs."""
    with torch.no_grad():
        _, ids = block.router.route(x_dev, block.expert_bias_E)
    ids = ids.cpu()
    E = spec.num_experts
    ok = stable_tokens(aux["logits"], spec, expert_bias)
    differ = ~(ids == aux["ids_TK"]).all(-1)
    note(f"block routing {label}: {int(differ.sum())} of {ids.shape[0]} tokens differ from the oracle, "
         f"{int((~ok).sum())} are near ties")
    assert ok.float().mean() > 0.97
    assert not differ[ok].any(), "routing differs on tokens that are not near ties"
    assert int(differ.sum()) <= int((~ok).sum())
    counters = block.tokens_per_expert_E.cpu().long()
    assert torch.equal(counters, torch.bincount(ids.reshape(-1), minlength=E)), \
        "tokens_per_expert_E is not the count of the routed ids"
    if not differ.any():
        assert torch.equal(counters, aux["counts_E"])
    else:  # a flipped token moves one assignment between two experts
        assert int((counters - aux["counts_E"]).abs().sum()) <= 2 * spec.top_k * int(differ.sum())
    return ids


@pytest.mark.parametrize("dispatcher,T", [("local", 1024), ("padded", 1536)])
def test_qwen3_shape_bf16_forward_backward(dispatcher, T):
    """hidden 2048, 128 experts, top-8, intermediate 768, softmax + norm, bf16; local dispatch,
    and 128-row padded dispatch under a Zipf(1.2)-shaped logit bias solved for a 60 % load share
    of the busiest fifth of the experts."""
    print(f"block qwen3 bf16 {dispatcher} T={T}", flush=True)
    D, E, K, F = 2048, 128, 8, 768
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=0)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0)).bfloat16()
    gout = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).bfloat16()
    if dispatcher == "padded":
        p.router_logit_bias_E, reached = zipf_logit_bias(x.float() @ p.router_w_ED.T, K, top20_share=0.60)
        assert abs(reached - 0.60) < 0.02
    kw = dict(dispatcher=dispatcher, pad_multiple=128) if dispatcher == "padded" else {}
    got, want, aux, block = _run_pair(p, spec, x, gout, torch.bfloat16, D, F, **kw)
    ids = _check_routing(block, x.to(DEV), aux, spec, label=dispatcher)
    if dispatcher == "padded":
        load = torch.bincount(ids.reshape(-1), minlength=E).sort(descending=True).values
        share = float(load[: E // 5].sum()) / (T * K)
        note(f"block padded T={T}: load histogram (sorted) max {int(load[0])}, median {int(load[E // 2])}, "
             f"min {int(load[-1])}; top-20% share {share:.3f}")
        assert 0.55 <= share <= 0.65
    for k in want:
        err = rel_l2(got[k], want[k])
        assert err < 2e-2, f"{k}: rel-L2 {err}"


@pytest.mark.parametrize("dtype,T,D,E,K,F,dispatcher", [
    (torch.float32, 300, 64, 8, 2, 96, "local"),
    (torch.bfloat16, 700, 512, 16, 4, 384, "local"),
    (torch.bfloat16, 900, 384, 16, 4, 640, "padded"),
    (torch.bfloat16, 700, 512, 16, 4, 384, "share"),
])
def test_block_with_the_situ_activation_matches_the_oracle(dtype, T, D, E, K, F, dispatcher):
    """Experts with SituGLU (activation.py:40-64) instead of SwiGLU: gate, up and down run as
    grouped linear maps with the module's own torch arithmetic between them.  The oracle calls
    the restated formula (oracle.moe_ref.situ_glu), not the package's module."""
    from torchllmtuner_amd import moe

    print(f"block situ {dtype} T={T} D={D} E={E} K={K} F={F} {dispatcher}", flush=True)
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True)
    kw = {}
    El = E
    if dispatcher == "padded":
        kw = dict(dispatcher="padded", pad_multiple=64)
    elif dispatcher == "share":
        kw = dict(dispatcher="share", local=(4, 12))
        El = 8
    p = make_params(E, D, F, dtype, seed=3, std=0.05, El=El)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0)).to(dtype)
    gout = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).to(dtype)
    beta, linear_beta = 2.0, 1.7
    leaves = {k: getattr(p, k).clone().requires_grad_() for k in ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF")}
    xr = x.clone().requires_grad_()
    okw = {}
    if dispatcher == "padded":
        okw["pad_multiple"] = 64
    if dispatcher == "share":
        okw["local_experts"] = (4, 12)
    ref, aux = R.moe_forward(xr, R.MoEParams(**leaves), spec,
                             activation=lambda g, u: R.situ_glu(g, u, beta, linear_beta), **okw)
    ref.backward(gout)
    block = build_block(p, spec, D, F, dtype, DEV, activation=moe.SituGLU(beta, linear_beta), **kw)
    assert not block.routed_experts.inner_experts.fuses_activation()
    xd = x.to(DEV).requires_grad_()
    out = block(xd)
    out.backward(gout.to(DEV))
    _check_routing(block, x.to(DEV), aux, spec, label="situ " + dispatcher)
    ie = block.routed_experts.inner_experts
    got = {"out": out, "dx": xd.grad, "router_w_ED": block.router.gate.weight.grad,
           "w1_EFD": ie.w1_EFD.grad, "w3_EFD": ie.w3_EFD.grad, "w2_EDF": ie.w2_EDF.grad}
    want = {"out": ref, "dx": xr.grad, **{k: v.grad for k, v in leaves.items()}}
    for k in want:
        if dtype == torch.float32:
            assert rel_max(got[k], want[k]) < 1e-5, f"{k}: {rel_max(got[k], want[k])}"
        else:
            assert rel_l2(got[k], want[k]) < 2e-2, f"{k}: rel-L2 {rel_l2(got[k], want[k])}"
    # and the same block with SwiGLU gives something else (the activation is really used)
    swi = build_block(p, spec, D, F, dtype, DEV, **kw)
    assert rel_l2(swi(x.to(DEV)), ref) > 5e-2


def test_deepseek_shape_local_share_with_shared_expert():
    """hidden 7168 scaled down in F only where the CPU oracle needs it: D=7168, 256
    experts, sigmoid + bias, 8 groups / 4 kept, top-8, scale 2.5, experts 0-31 local,
    one shared expert.  F=512 keeps the CPU side to seconds."""
    print("block deepseek share", flush=True)
    T, D, E, K, F = 512, 7168, 256, 8, 512
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True, route_scale=2.5,
                        num_expert_groups=8, num_limited_groups=4)
    p = make_params(E, D, F, torch.bfloat16, seed=0, shared_F=F, El=32)
    p.expert_bias_E = torch.rand(E, generator=torch.Generator().manual_seed(2)) * 0.2 - 0.1
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0)).bfloat16()
    gout = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).bfloat16()
    got, want, aux, block = _run_pair(p, spec, x, gout, torch.bfloat16, D, F, dispatcher="share", local=(0, 32))
    _check_routing(block, x.to(DEV), aux, spec, p.expert_bias_E, label="deepseek share")
    # counts cover all 256 experts although only 32 are computed
    assert int(block.tokens_per_expert_E.sum().item()) == T * K
    for k in want:
        err = rel_l2(got[k], want[k])
        assert err < 2e-2, f"{k}: rel-L2 {err}"


def test_block_api_contract():
    """Shapes, (B,S,D) handling, eval mode leaves counters alone, router-logits arity,
    padding mask filters only the statistics, bias update closed form."""
    print("block api", flush=True)
    D, E, K, F = 64, 8, 2, 64
    spec = R.RouterSpec(E, K, score_func="sigmoid")
    p = make_params(E, D, F, torch.float32, seed=3, std=0.2)
    block = build_block(p, spec, D, F, torch.float32, DEV, load_balance_coeff=1e-3)
    x = torch.randn(2, 5, D, device=DEV)
    block.eval()
    out = block(x)
    assert out.shape == x.shape and block.tokens_per_expert_E.sum() == 0
    block.train()
    mask = torch.zeros(2, 5, dtype=torch.bool, device=DEV)
    mask[1, 3:] = True
    out_m = block(x, padding_mask=mask)
    assert torch.equal(out_m, out), "padding mask must not change the output"
    assert int(block.tokens_per_expert_E.sum().item()) == 8 * K
    block.set_padding_mask(None)
    block.tokens_per_expert_E.zero_()
    block(x)
    assert int(block.tokens_per_expert_E.sum().item()) == 10 * K
    # bias update: bias += c*sign(mean - counts) - mean(.)   (layer.py:204-228)
    counts = block.tokens_per_expert_E.clone()
    block.update_expert_bias()
    delta = 1e-3 * torch.sign(counts.mean() - counts)
    torch.testing.assert_close(block.expert_bias_E, delta - delta.mean())
    assert block.tokens_per_expert_E.sum() == 0
    block.returns_router_logits = True
    o2 = block(x)
    assert isinstance(o2, tuple) and o2[1] is None
    with pytest.raises(ValueError, match="dtype bool"):
        block(x, padding_mask=torch.zeros(2, 5, device=DEV))
    assert [k for k in block.state_dict()] == [
        "expert_bias_E", "routed_experts.inner_experts.w1_EFD", "routed_experts.inner_experts.w3_EFD",
        "routed_experts.inner_experts.w2_EDF", "router.gate.weight"]


@pytest.mark.parametrize("T", [0, 3])
def test_bf16_block_with_no_or_few_tokens(T):
    """The MFMA path with nothing or almost nothing to do: no tokens at all (every weight
    gradient is zeros, dx is empty) and three tokens (most experts have no rows)."""
    print(f"block bf16 edge T={T}", flush=True)
    D, E, K, F = 384, 16, 2, 384
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=5)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(0)).bfloat16()
    gout = torch.randn(T, D, generator=torch.Generator().manual_seed(1)).bfloat16()
    got, want, aux, block = _run_pair(p, spec, x, gout, torch.bfloat16, D, F)
    assert got["out"].shape == (T, D)
    ie = block.routed_experts.inner_experts
    for w in (ie.w1_EFD, ie.w3_EFD, ie.w2_EDF, block.router.gate.weight):
        assert w.grad is not None and bool(torch.isfinite(w.grad.float()).all())
    if T == 0:
        for w in (ie.w1_EFD, ie.w3_EFD, ie.w2_EDF):
            assert not bool(w.grad.any())
        return
    counts = aux["counts_E"]
    unused = (counts == 0).nonzero().squeeze(-1)
    assert unused.numel() >= E - T * K
    for w in (ie.w1_EFD, ie.w3_EFD, ie.w2_EDF):
        assert not bool(w.grad[unused.to(DEV)].any()), "experts without rows get zero gradients"
    for k in want:
        err = rel_l2(got[k], want[k])
        assert err < 2e-2, f"{k}: rel-L2 {err}"


def test_forward_without_gradients_skips_gate_and_up_and_returns_the_same_bits():
    """Under no_grad the fused forward does not write gate and up (nobody will read them); the
    block's output must not change by a bit, and a differentiated forward right after still works."""
    print("block forward only", flush=True)
    T, D, E, K, F = 700, 512, 16, 4, 384
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=21)
    block = build_block(p, spec, D, F, torch.bfloat16, DEV)
    x = torch.randn(T, D, generator=torch.Generator().manual_seed(22)).bfloat16().to(DEV)
    block.eval()
    with torch.no_grad():
        plain = block(x)
    xin = x.clone().requires_grad_()
    tracked = block(xin)
    assert torch.equal(plain, tracked)
    tracked.float().sum().backward()
    assert torch.isfinite(xin.grad.float()).all() and float(xin.grad.float().abs().sum()) > 0


@pytest.mark.parametrize("dtype,D,F,dispatcher,shared_F", [
    (torch.float32, 256, 512, "local", None), (torch.bfloat16, 512, 384, "local", None),
    (torch.bfloat16, 384, 512, "padded", None),
    # with a shared expert: it runs on the library's second stream, a fork and join inside the graph
    (torch.bfloat16, 512, 384, "local", 448), (torch.float32, 128, 192, "local", 64)])
def test_block_step_replays_from_a_hip_graph(dtype, D, F, dispatcher, shared_F):
    """Forward + backward of the block captured once as a HIP graph: no kernel of the path
    synchronises the host, reads a size back or allocates outside PyTorch's allocator, so the
    whole step captures as it is.  Every replay -- with eager steps and synchronisations between
    them, and with new token values in the captured input buffer -- must reproduce the eager
    step's output and gradients bit for bit (the kernels use no atomics)."""
    print(f"block under a HIP graph {dtype} D={D} F={F} {dispatcher} shared={shared_F}", flush=True)
    T, E, K = 600, 16, 4
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, dtype, seed=31, shared_F=shared_F)
    kw = dict(pad_multiple=64) if dispatcher == "padded" else {}
    block = build_block(p, spec, D, F, dtype, DEV, dispatcher=dispatcher, **kw)
    block.train()
    g = torch.Generator().manual_seed(32)
    xin = torch.randn(T, D, generator=g).to(dtype).to(DEV).requires_grad_()
    gout = torch.randn(T, D, generator=g).to(dtype).to(DEV)
    params = [q for q in block.parameters() if q.requires_grad]

    def step():
        return torch.autograd.grad(block(xin), [xin] + params, gout)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for rep in range(3):
        with torch.no_grad():
            xin.copy_(torch.randn(T, D, generator=g).to(dtype))  # new tokens, new routing
        eager = [t.clone() for t in step()]
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for got, want in zip(captured, eager):
            assert torch.equal(got, want), f"replay {rep} differs from the eager step"


def test_shared_expert_on_the_second_stream_gives_the_one_stream_results():
    """A block with a shared expert, run with the shared expert on the library's second stream and
    with everything on the caller's stream: the same output and parameter gradients bit for bit
    (the input gradient sums its three parts in another order: one bf16 rounding), several steps in
    a row, also on a caller's own stream, with the results consumed at once."""
    print("block shared expert on a second stream", flush=True)
    T, D, E, K, F, Fs = 1500, 512, 16, 4, 384, 640
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=5, std=0.05, shared_F=Fs)
    block = build_block(p, spec, D, F, torch.bfloat16, DEV)
    block.train()
    g = torch.Generator().manual_seed(6)
    x = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    gout = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    params = [q for q in block.parameters() if q.requires_grad]

    def step():
        xin = x.detach().clone().requires_grad_()
        out = block(xin)
        grads = torch.autograd.grad(out, [xin] + params, gout)
        # (detached: a graph kept alive would keep the parameters' gradient accumulators of this
        # step, with this step's stream, for the next one)
        return [out.detach()] + [t.clone() for t in grads]

    block.overlap_shared_experts = False
    want = step()
    torch.cuda.synchronize()
    block.overlap_shared_experts = True
    from torchllmtuner_amd import ops
    assert ops.aux_stream(x.device) is not None
    mine = torch.cuda.Stream()
    for stream in (torch.cuda.current_stream(), mine):
        stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(stream):
            for it in range(4):
                got = step()
                assert torch.equal(got[0], want[0]), f"out, step {it}"
                assert rel_l2(got[1], want[1]) < 4e-3, f"dx, step {it}"
                for a, b in zip(got[2:], want[2:]):
                    assert torch.equal(a, b), f"parameter gradient, step {it}"
        torch.cuda.current_stream().wait_stream(stream)
    torch.cuda.synchronize()
    # without gradients too
    with torch.no_grad():
        assert torch.equal(block(x), want[0])


def _random_case(rng):
    dtype = rng.choice([torch.float32, torch.bfloat16])
    T = rng.choice([1, 2, 7, 64, 130, 257, 600])
    D = rng.choice([64, 96, 128, 384, 448, 512])
    F = rng.choice([64, 128, 384, 576, 640])
    E = rng.choice([2, 5, 8, 64])
    K = rng.choice([k for k in (1, 2, 3, 6) if k <= E])
    spec = R.RouterSpec(E, K, score_func=rng.choice(["softmax", "sigmoid", "sqrtsoftplus"]),
                        route_norm=rng.choice([True, False]), route_scale=rng.choice([1.0, 2.5]))
    kind = rng.choice(["local", "padded", "share", "local"])
    kw, El = {}, E
    if kind == "padded":
        kw = dict(dispatcher="padded", pad_multiple=rng.choice([1, 8, 128]))
    elif kind == "share":
        lo = rng.randrange(0, E - 1)
        hi = rng.randrange(lo + 1, E + 1)
        kw, El = dict(dispatcher="share", local=(lo, hi)), hi - lo
    batch = rng.choice([True, False]) and T % 2 == 0
    return dtype, T, D, F, E, K, spec, kw, El, batch


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_randomised_small_shapes_match_the_oracle(seed):
    """Sixteen seeded random configurations per seed -- dtype, token count (down to one token),
    widths on and off the MFMA path, expert count, top-k, score function, norm, scale, dispatcher
    (local, padded, one rank's share), flat or (B, S, D) input -- forward and every gradient
    against the oracle.  A token whose choice is a few-ulp near tie may flip; then only the
    routing bound is checked for that case."""
    import random

    rng = random.Random(seed)
    for it in range(16):
        dtype, T, D, F, E, K, spec, kw, El, batch = _random_case(rng)
        print(f"block random case {seed}/{it}: {dtype} T={T} D={D} F={F} E={E} K={K} {spec.score_func} "
              f"norm={spec.route_norm} scale={spec.route_scale} {kw} batch={batch}", flush=True)
        p = make_params(E, D, F, dtype, seed=100 * seed + it, std=0.05, El=El)
        g = torch.Generator().manual_seed(1000 * seed + it)
        shape = (2, T // 2, D) if batch else (T, D)
        x = torch.randn(*shape, generator=g).to(dtype)
        gout = torch.randn(*shape, generator=g).to(dtype)
        got, want, aux, block = _run_pair(p, spec, x, gout, dtype, D, F, **kw)
        ok = stable_tokens(aux["logits"], spec)
        with torch.no_grad():
            _, ids = block.router.route(x.reshape(-1, D).to(DEV), block.expert_bias_E)
        differ = ~(ids.cpu() == aux["ids_TK"]).all(-1)
        assert not differ[ok].any(), "routing differs on tokens that are not near ties"
        if differ.any():
            continue
        for k in want:
            gm, wm = float(got[k].detach().float().abs().max()), float(want[k].detach().float().abs().max())
            if k == "router_w_ED" and K == 1 and spec.route_norm and max(gm, wm) < 1e-4:
                continue  # d/ds of s / (s + 1e-20) is zero: both sides hold rounding noise only
            if wm == 0.0:
                assert gm == 0.0, k
                continue
            err = rel_max(got[k], want[k]) if dtype == torch.float32 else rel_l2(got[k].float(), want[k].float())
            assert err < (1e-5 if dtype == torch.float32 else 2e-2), f"{k}: {err}"


def test_dispatcher_api_matches_reference_contract():
    """dispatch/combine through the public dispatcher classes, analytic expectation
    out = x * 2 * sum(scores) (tests/unit_tests/cpu/models/test_moe_token_dispatch.py:249-309)."""
    print("dispatcher api", flush=True)
    from torchllmtuner_amd import moe

    g = torch.Generator().manual_seed(0)
    x = torch.randn(6, 4, generator=g)
    ids = torch.randint(0, 4, (6, 2), generator=g)
    sc = torch.rand(6, 2, generator=g)
    counts = torch.bincount(ids.reshape(-1), minlength=4)
    want = x * (2 * sc.sum(-1, keepdim=True))
    for disp in (moe.LocalTokenDispatcher(4, 2), moe.PaddedTokenDispatcher(4, 2, pad_multiple=4)):
        xd = x.to(DEV).requires_grad_()
        sd = sc.to(DEV).requires_grad_()
        routed, out_counts, meta = disp.dispatch(xd, sd, ids.to(DEV), counts.to(DEV))
        if isinstance(disp, moe.PaddedTokenDispatcher):
            assert out_counts.tolist() == [int(c) + (-int(c) % 4) for c in counts.tolist()]
            assert routed.shape[0] == int(out_counts.sum())
        else:
            assert routed.shape == (12, 4)
            assert torch.equal(meta.token_indices_experts_sorted_N.cpu(),
                               torch.argsort(ids.reshape(-1), stable=True) // 2)
        out = disp.combine(routed * 2.0, meta, xd)
        torch.testing.assert_close(out.cpu(), want)
        out.sum().backward()
        torch.testing.assert_close(xd.grad.cpu(), (2 * sc.sum(-1, keepdim=True)).expand_as(x))
        torch.testing.assert_close(sd.grad.cpu(), (2 * x.sum(-1, keepdim=True)).expand_as(sc))
    with pytest.raises(ValueError, match="token count and top_k"):
        moe.LocalTokenDispatcher(4, 2).dispatch(torch.ones(2, 3, device=DEV), torch.ones(3, 2, device=DEV),
                                                torch.zeros(2, 2, dtype=torch.long, device=DEV), counts.to(DEV))
    with pytest.raises(RuntimeError, match="no CPU implementation"):
        moe.LocalTokenDispatcher(4, 2).dispatch(x, sc, ids, counts)


def test_full_size_properties_qwen3_t8192():
    """The benchmark's own size (T=8192, D=2048, E=128, K=8, F=768, bf16), too large for the
    CPU oracle: size-independent properties instead.

    * the plan is a permutation of the T*K slots, counts add up, every row maps back;
    * scaling w2 by 2 (exact in bf16) scales the output by exactly 2, bit for bit;
    * a sample of tokens recomputed token by token in fp32 on the device agrees within
      the bf16 bar; a sample of experts' weight gradients recomputed from the same
      intermediates with plain matmuls agrees within it too;
    * two runs give bit-identical outputs and gradients (no atomics anywhere).
    """
    print("block full size T=8192", flush=True)
    from torchllmtuner_amd import ops

    T, D, E, K, F = 8192, 2048, 128, 8, 768
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=3)
    block = build_block(p, spec, D, F, torch.bfloat16, DEV)
    block.train()
    g = torch.Generator().manual_seed(4)
    x = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    gout = torch.randn(T, D, generator=g).bfloat16().to(DEV)

    def run():
        block.zero_grad(set_to_none=True)
        xin = x.clone().requires_grad_()
        out = block(xin)
        out.backward(gout)
        ie = block.routed_experts.inner_experts
        return out.detach(), xin.grad, ie.w1_EFD.grad.clone(), ie.w3_EFD.grad.clone(), ie.w2_EDF.grad.clone(), \
            block.router.gate.weight.grad.clone()

    first = run()
    second = run()
    for a, b in zip(first, second):
        assert torch.equal(a, b), "two runs on the same inputs differ"
    out, dx, dw1, dw3, dw2, dwr = first
    for t in first:
        assert torch.isfinite(t.float()).all()

    # --- plan: permutation, counts
    with torch.no_grad():
        scores, ids = block.router.route(x)
        plan = block.routed_experts.token_dispatcher.plan(ids)
    N = T * K
    assert int(plan.counts_E.sum()) == N and int(plan.total_rows) == N
    ros = plan.row_of_slot.long()
    assert torch.equal(torch.sort(ros).values, torch.arange(N, device=DEV))
    assert torch.equal(plan.slot_of_row.long()[ros], torch.arange(N, device=DEV))
    assert torch.equal(plan.token_of_row.long(), plan.slot_of_row.long() // K)
    sorted_ids = ids.reshape(-1)[plan.slot_of_row.long()]
    assert bool((sorted_ids[1:] >= sorted_ids[:-1]).all()), "rows are not expert-major"
    assert torch.equal(torch.bincount(ids.reshape(-1), minlength=E).int(), plan.counts_E)
    assert bool((ids.sort(-1).values[:, 1:] != ids.sort(-1).values[:, :-1]).all()), "an expert chosen twice"

    # --- exact linearity in w2 (power-of-two scaling commutes with every rounding)
    ie = block.routed_experts.inner_experts
    with torch.no_grad():
        ie.w2_EDF.mul_(2.0)
        out2 = block(x)
        ie.w2_EDF.mul_(0.5)
    assert torch.equal(out2, out * 2), "output is not exactly linear in w2"

    # --- sampled tokens, recomputed one by one in fp32 on the device
    w1, w3, w2 = ie.w1_EFD.detach(), ie.w3_EFD.detach(), ie.w2_EDF.detach()
    sample = torch.randint(0, T, (48,), generator=g).tolist()
    ref = torch.zeros(len(sample), D, device=DEV)
    bf = lambda v: v.bfloat16().float()
    for i, t in enumerate(sample):
        xt = x[t].float()
        for k in range(K):
            e = int(ids[t, k])
            gate, up = bf(w1[e].float() @ xt), bf(w3[e].float() @ xt)
            h = bf(bf(torch.nn.functional.silu(gate)) * up)
            ref[i] += float(scores[t, k]) * bf(w2[e].float() @ h)
    assert rel_l2(out[sample].float(), ref) < 2e-2

    # --- sampled experts: weight gradients recomputed from x, ids, scores and gout alone
    _expert_weight_gradient_check(x, gout, ids, scores, w1, w3, w2, dw1, dw3, dw2, (0, 57, 127))
    # --- routing-score gradient: the device's against <y, dout> recomputed from the inputs, then
    # dW_router from fp32 autograd over the router path with the device's score gradient upstream
    with torch.no_grad():
        rows = ops.permute_rows_fwd(x, plan)
        y, _, _, _ = ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)
        _, dsc = ops.combine_bwd(gout, y, scores, plan)
    want = _score_gradient_reference(x, gout, ids, w1, w3, w2, sample[:8])
    assert bool(((dsc[sample[:8]] - want).abs() <= 2e-2 * want.abs().clamp_min(1.0)).all())
    _router_weight_gradient_check(block, x, ids, dsc, dwr, spec, (0, 3, 17, 40, 57, 88, 101, 127))


def _sampled_token_reference(x, ids, weights, w1, w3, w2, sample, lo=0, hi=None):
    """Token-by-token fp32 recomputation on the device with the bf16 rounding points of the
    expert MLP; experts outside [lo, hi) contribute nothing (one rank's share)."""
    bf = lambda v: v.bfloat16().float()
    hi = w1.shape[0] + lo if hi is None else hi
    ref = torch.zeros(len(sample), x.shape[1], device=x.device)
    for i, t in enumerate(sample):
        xt = x[t].float()
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            if not lo <= e < hi:
                continue
            gate, up = bf(w1[e - lo].float() @ xt), bf(w3[e - lo].float() @ xt)
            h = bf(bf(torch.nn.functional.silu(gate)) * up)
            ref[i] += float(weights[t, k]) * bf(w2[e - lo].float() @ h)
    return ref


def _expert_weight_gradient_check(x, gout, ids, scores, w1, w3, w2, dw1, dw3, dw2, experts, lo=0):
    """Weight gradients of the sampled local experts recomputed from the block's INPUTS alone --
    tokens, output gradient, the device's ids and routing scores, the weights -- with plain fp32
    torch ops on the device and the bf16 rounding points of the reference's op sequence; no
    intermediate of the kernels under test (rows, gate, up, h, dy) is read.  The rows of expert e
    are its slots in ascending order (the stable expert-major order), row r stands for token
    slot // K, and dy[r] = score[slot] * gout[token] (the combine's backward).  An expert without
    rows must get zeros."""
    bf = lambda v: v.bfloat16().float()
    K = ids.shape[1]
    flat_ids, flat_scores = ids.reshape(-1), scores.reshape(-1).float()
    for e in experts:
        slots = (flat_ids == e + lo).nonzero().squeeze(-1)
        if slots.numel() == 0:
            for dw in (dw1, dw3, dw2):
                assert not dw[e].any(), f"expert {e + lo} has no rows but a gradient"
            continue
        tok = slots // K
        rows = x[tok].float()
        gf, uf = bf(rows @ w1[e].float().T), bf(rows @ w3[e].float().T)
        sig = torch.sigmoid(gf)
        silu = bf(gf * sig)
        h = bf(silu * uf)
        dyf = bf(flat_scores[slots][:, None] * gout[tok].float())
        dh = bf(dyf @ w2[e].float())
        dup = bf(dh * silu)
        dgate = bf(bf(dh * uf) * (sig * (1 + gf * (1 - sig))))
        for name, got, want in (("dw2", dw2[e], dyf.T @ h), ("dw1", dw1[e], dgate.T @ rows), ("dw3", dw3[e], dup.T @ rows)):
            err = rel_l2(got.float(), want)
            assert err < 2e-2, f"{name}[{e + lo}] ({slots.numel()} rows): rel-L2 {err}"


def _score_gradient_reference(x, gout, ids, w1, w3, w2, tokens, lo=0, hi=None):
    """d out / d score[t, k] = <y(t, k), gout[t]> for the given tokens, y recomputed from the token
    and the weights in fp32 with the expert MLP's bf16 rounding points (zero for experts outside
    [lo, hi): their rows are not computed here)."""
    bf = lambda v: v.bfloat16().float()
    hi = w1.shape[0] + lo if hi is None else hi
    want = torch.zeros(len(tokens), ids.shape[1], device=x.device)
    for i, t in enumerate(tokens):
        xt = x[t].float()
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            if not lo <= e < hi:
                continue
            gate, up = bf(w1[e - lo].float() @ xt), bf(w3[e - lo].float() @ xt)
            h = bf(bf(torch.nn.functional.silu(gate)) * up)
            want[i, k] = (bf(w2[e - lo].float() @ h) * gout[t].float()).sum()
    return want


def _router_weight_gradient_check(block, x, ids, dscore, dwr, spec, experts):
    """dW_router from fp32 autograd over the router path alone -- gate (+ logit bias), score
    function, gather at the device's ids, norm, scale -- with the device's routing-score gradient
    as the upstream gradient; the rows of the sampled experts and the whole matrix."""
    wr = block.router.gate.weight.detach().float().clone().requires_grad_()
    lb = None if block.router.gate.bias is None else block.router.gate.bias.detach().float()
    logits = x.float() @ wr.T + (0 if lb is None else lb)
    s = torch.softmax(logits, -1) if spec.score_func == "softmax" else torch.sigmoid(logits)
    w = s.gather(-1, ids)
    if spec.route_norm:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    (w * spec.route_scale * dscore.float()).sum().backward()
    for e in experts:
        err = rel_l2(dwr[e].float(), wr.grad[e])
        assert err < 2e-2, f"dW_router[{e}]: rel-L2 {err}"
    assert rel_l2(dwr.float(), wr.grad) < 2e-2


def _token_gradient_reference(block, x, gout, ids, sample, spec, lo=0, hi=None):
    """out[t] and d<out[t], gout[t]>/dx[t] of the sampled tokens by fp32 autograd on the device,
    one token at a time, with the device's ids held fixed: router gate (+ logit bias), score
    function, gather, norm, scale, the chosen local experts, the shared expert."""
    ie = block.routed_experts.inner_experts
    w1, w3, w2 = (w.detach().float() for w in (ie.w1_EFD, ie.w3_EFD, ie.w2_EDF))
    hi = w1.shape[0] + lo if hi is None else hi
    wr = block.router.gate.weight.detach().float()
    lb = None if block.router.gate.bias is None else block.router.gate.bias.detach().float()
    sh = block.shared_experts
    silu = torch.nn.functional.silu
    outs, grads = [], []
    for t in sample:
        xt = x[t].float().clone().requires_grad_()
        logits = wr @ xt + (0 if lb is None else lb)
        s = torch.softmax(logits, -1) if spec.score_func == "softmax" else torch.sigmoid(logits)
        w = s[ids[t]]
        if spec.route_norm:
            w = w / (w.sum() + 1e-20)
        w = w * spec.route_scale
        out = torch.zeros_like(xt)
        for k in range(ids.shape[1]):
            e = int(ids[t, k])
            if lo <= e < hi:
                out = out + w[k] * (w2[e - lo] @ (silu(w1[e - lo] @ xt) * (w3[e - lo] @ xt)))
        if sh is not None:
            sg, su, sd = (m.weight.detach().float() for m in (sh.gate_proj, sh.up_proj, sh.down_proj))
            out = out + sd @ (silu(sg @ xt) * (su @ xt))
        (out * gout[t].float()).sum().backward()
        outs.append(out.detach())
        grads.append(xt.grad)
    return torch.stack(outs), torch.stack(grads)


def test_full_size_properties_skewed_padded_t16384():
    """T=16384 at the Qwen3 shape, skewed routing (Zipf(1.2)-shaped logit bias solved for a 60 %
    load share of the busiest fifth, one expert switched off entirely), 128-row padded segments:
    the load histogram, layout invariants of the padded plan, determinism, and -- against plain
    fp32 recomputation on the device -- sampled tokens' outputs and input gradients, the weight
    gradients of the hottest, the coldest and the empty expert, and sampled routing-score dots."""
    print("block full size padded T=16384", flush=True)
    from torchllmtuner_amd import ops

    T, D, E, K, F = 16384, 2048, 128, 8, 768
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, torch.bfloat16, seed=5)
    g = torch.Generator().manual_seed(6)
    x_cpu = torch.randn(T, D, generator=g).bfloat16()
    gout = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    bias, reached = zipf_logit_bias(x_cpu[:4096].float() @ p.router_w_ED.T, K, top20_share=0.60)
    bias[E - 1] = -1e4  # nobody chooses the last expert: a zero-row segment at full size
    p.router_logit_bias_E = bias
    x = x_cpu.to(DEV)
    block = build_block(p, spec, D, F, torch.bfloat16, DEV, dispatcher="padded", pad_multiple=128)
    block.train()

    def run():
        block.zero_grad(set_to_none=True)
        xin = x.clone().requires_grad_()
        out = block(xin)
        out.backward(gout)
        ie = block.routed_experts.inner_experts
        return out.detach(), xin.grad, ie.w1_EFD.grad.clone(), ie.w3_EFD.grad.clone(), ie.w2_EDF.grad.clone(), \
            block.router.gate.weight.grad.clone()

    first, second = run(), run()
    for a, b in zip(first, second):
        assert torch.equal(a, b) and torch.isfinite(a.float()).all()
    out, dx, dw1, dw3, dw2, dwr = first
    with torch.no_grad():
        scores, ids = block.router.route(x)
        plan = block.routed_experts.token_dispatcher.plan(ids)
    counts = torch.bincount(ids.reshape(-1), minlength=E)
    assert torch.equal(plan.counts_E.long(), counts)
    assert torch.equal(block.tokens_per_expert_E.long(), 2 * counts)  # two training forwards
    top = counts.sort(descending=True).values
    share = float(top[: E // 5].sum()) / (T * K)
    note(f"block full size T=16384 skewed: rows per expert (sorted) {top[:4].tolist()} ... median {int(top[E // 2])} "
         f"... {top[-4:].tolist()}; top-20% share {share:.3f} (solved on 4096 tokens: {reached:.3f})")
    assert 0.55 <= share <= 0.65, "the load is not the stated skew"
    assert int(counts[E - 1]) == 0
    padded = plan.seg_offsets[1:] - plan.seg_offsets[:-1]
    assert torch.equal(padded.long(), counts + (-counts % 128))
    total = int(plan.total_rows)
    sor = plan.slot_of_row[:total].long()
    real = sor >= 0
    assert int(real.sum()) == T * K
    assert torch.equal(torch.sort(sor[real]).values, torch.arange(T * K, device=DEV))
    # padding sits at the end of each segment
    off = plan.seg_offsets.long()
    e_of_row = torch.bucketize(torch.arange(total, device=DEV), off[1:], right=True)
    within = torch.arange(total, device=DEV) - off[e_of_row]
    assert torch.equal(real, within < counts.to(DEV)[e_of_row])

    ie = block.routed_experts.inner_experts
    w1, w3, w2 = ie.w1_EFD.detach(), ie.w3_EFD.detach(), ie.w2_EDF.detach()
    sample = torch.randint(0, T, (12,), generator=g).tolist()
    ref_out, ref_dx = _token_gradient_reference(block, x, gout, ids, sample, spec)
    assert rel_l2(out[sample].float(), ref_out) < 2e-2
    assert rel_l2(dx[sample].float(), ref_dx) < 2e-2
    hottest, coldest = int(counts.argmax()), int(counts[: E - 1].argmin())
    _expert_weight_gradient_check(x, gout, ids, scores, w1, w3, w2, dw1, dw3, dw2, (hottest, 40, coldest, E - 1))
    with torch.no_grad():
        rows = ops.permute_rows_fwd(x, plan)
        y, _, _, _ = ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)
        _, dsc = ops.combine_bwd(gout, y, scores, plan)
    want = _score_gradient_reference(x, gout, ids, w1, w3, w2, sample[:6])
    assert bool(((dsc[sample[:6]] - want).abs() <= 2e-2 * want.abs().clamp_min(1.0)).all())
    _router_weight_gradient_check(block, x, ids, dsc, dwr, spec, (hottest, 1, 9, 40, 77, 100, coldest, 120))


def test_full_size_properties_deepseek_local_share():
    """The DeepSeek-V3-shaped block at full size: T=4096, D=7168, 256 experts in 8 groups
    (4 kept), sigmoid + bias, top-8, scale 2.5, F=2048, experts 0-31 computed here, one
    shared expert of width 2048.  Group confinement, full-E statistics, and -- against plain fp32
    recomputation on the device -- sampled tokens' outputs and input gradients, sampled local
    experts' weight gradients at F=2048, and the shared expert's weight gradients."""
    print("block full size deepseek share", flush=True)
    from torchllmtuner_amd import ops

    T, D, E, K, F = 4096, 7168, 256, 8, 2048
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True, route_scale=2.5,
                        num_expert_groups=8, num_limited_groups=4)
    p = make_params(E, D, F, torch.bfloat16, seed=7, shared_F=F, El=32)
    p.expert_bias_E = torch.rand(E, generator=torch.Generator().manual_seed(2)) * 0.2 - 0.1
    block = build_block(p, spec, D, F, torch.bfloat16, DEV, load_balance_coeff=1e-3, dispatcher="share", local=(0, 32))
    block.train()
    g = torch.Generator().manual_seed(8)
    x = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    gout = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    xin = x.clone().requires_grad_()
    out = block(xin)
    out.backward(gout)
    out, dx = out.detach(), xin.grad
    assert torch.isfinite(out.float()).all() and torch.isfinite(dx.float()).all()
    assert int(block.tokens_per_expert_E.sum().item()) == T * K
    with torch.no_grad():
        scores, ids = block.router.route(x, block.expert_bias_E)
        plan = block.routed_experts.token_dispatcher.plan(ids)
    assert torch.equal(block.tokens_per_expert_E.long(), torch.bincount(ids.reshape(-1), minlength=E))
    groups = ids // 32
    assert int(max(len(set(r)) for r in groups.cpu().tolist())) <= 4, "a token left its 4 groups"
    assert bool((ids.sort(-1).values[:, 1:] != ids.sort(-1).values[:, :-1]).all())
    torch.testing.assert_close(scores.sum(-1), torch.full((T,), 2.5, device=DEV), rtol=1e-5, atol=1e-5)
    local_rows = int((ids < 32).sum())
    assert 0 < local_rows < T * K and int(plan.total_rows) == local_rows

    ie = block.routed_experts.inner_experts
    w1, w3, w2 = ie.w1_EFD.detach(), ie.w3_EFD.detach(), ie.w2_EDF.detach()
    # tokens with at least one local expert first, so the routed part of the check is not vacuous
    has_local = (ids < 32).any(-1).nonzero().squeeze(-1)
    sample = has_local[torch.randint(0, has_local.numel(), (8,), generator=g)].tolist() + \
        torch.randint(0, T, (4,), generator=g).tolist()
    ref_out, ref_dx = _token_gradient_reference(block, x, gout, ids, sample, spec, lo=0, hi=32)
    assert rel_l2(out[sample].float(), ref_out) < 2e-2
    assert rel_l2(dx[sample].float(), ref_dx) < 2e-2
    lc = plan.seg_counts.cpu()
    _expert_weight_gradient_check(x, gout, ids, scores, w1, w3, w2, ie.w1_EFD.grad, ie.w3_EFD.grad,
                                  ie.w2_EDF.grad, (int(lc.argmax()), 7, int(lc.argmin())))
    with torch.no_grad():
        rows = ops.permute_rows_fwd(x, plan)
        y, _, _, _ = ops.grouped_swiglu_fwd(rows, w1, w3, w2, plan)
        _, dsc = ops.combine_bwd(gout, y, scores, plan)
    want = _score_gradient_reference(x, gout, ids, w1, w3, w2, sample[:6], lo=0, hi=32)
    assert bool(((dsc[sample[:6]] - want).abs() <= 2e-2 * want.abs().clamp_min(1.0)).all())
    _router_weight_gradient_check(block, x, ids, dsc, block.router.gate.weight.grad, spec,
                                  (0, 5, 31, 32, 100, 177, 200, 255))
    # the shared expert: a dense SwiGLU over all tokens, gradients from plain fp32 matmuls
    sh = block.shared_experts
    bf = lambda v: v.bfloat16().float()
    xf, gf_ = x.float(), gout.float()
    gate, up = bf(xf @ sh.gate_proj.weight.float().T), bf(xf @ sh.up_proj.weight.float().T)
    sig = torch.sigmoid(gate)
    h = bf(bf(gate * sig) * up)
    dh = bf(gf_ @ sh.down_proj.weight.float())
    dup = bf(dh * bf(gate * sig))
    dgate = bf(bf(dh * up) * (sig * (1 + gate * (1 - sig))))
    for name, got, want in (("shared down", sh.down_proj.weight.grad, gf_.T @ h),
                            ("shared gate", sh.gate_proj.weight.grad, dgate.T @ xf),
                            ("shared up", sh.up_proj.weight.grad, dup.T @ xf)):
        err = rel_l2(got.float(), want)
        assert err < 2e-2, f"{name}: rel-L2 {err}"


@pytest.mark.parametrize("score_func,with_padding", [("sigmoid", True), ("softmax", False)])
def test_balance_loss_hook_injects_the_reference_gradient(score_func, with_padding):
    """An attached MicrobatchWiseLoadBalanceLoss adds coeff / tokens * d(sum f p) to the
    router's gradient path and accumulates its metric; fp32 so the bar is 1e-5."""
    print(f"block aux loss {score_func}", flush=True)
    from torchllmtuner_amd import moe

    T, D, E, K, F = 320, 128, 8, 2, 64
    coeff, denom = 3000.0, 300.0  # large on purpose: the aux term must be visible next to the main gradient
    spec = R.RouterSpec(E, K, score_func=score_func, route_norm=True)
    p = make_params(E, D, F, torch.float32, seed=11, std=0.1)
    g = torch.Generator().manual_seed(12)
    x = torch.randn(T, D, generator=g)
    gout = torch.randn(T, D, generator=g)
    pad = (torch.rand(T, generator=g) < 0.15) if with_padding else None

    leaves = {k: getattr(p, k).clone().requires_grad_() for k in ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF")}
    xr = x.clone().requires_grad_()
    ref, aux = R.moe_forward(xr, R.MoEParams(**leaves), spec)
    rmap = R.routing_map(aux["ids_TK"], E)
    if pad is not None:
        rmap = rmap & ~pad[:, None]
    raw = R.balance_loss(R.score(aux["logits"], score_func), rmap, pad)
    ((ref * gout).sum() + raw * (coeff / denom)).backward()

    block = build_block(p, spec, D, F, torch.float32, DEV)
    block.router.aux_loss = moe.MicrobatchWiseLoadBalanceLoss(coeff=coeff).to(DEV)
    block.train()
    moe.AuxLoss.set_step_denominator(torch.tensor(denom), model_parts=[block])
    xd = x.to(DEV).requires_grad_()
    out = block(xd, padding_mask=None if pad is None else pad.to(DEV))
    out.backward(gout.to(DEV))
    assert rel_max(out, ref) < 1e-5
    assert abs(float(block.router.aux_loss.instance_acc) - float(raw.detach()) / denom) < 1e-5 * max(1.0, float(raw.detach()) / denom)
    assert rel_max(block.router.gate.weight.grad, leaves["router_w_ED"].grad) < 1e-5
    assert rel_max(xd.grad, xr.grad) < 1e-5
    # and it is the aux term that moved the router gradient
    block.zero_grad(set_to_none=True)
    block.router.aux_loss = None
    xd2 = x.to(DEV).requires_grad_()
    block(xd2).backward(gout.to(DEV))
    assert rel_max(block.router.gate.weight.grad, leaves["router_w_ED"].grad) > 1e-4


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,D,F", [(torch.float32, 64, 96), (torch.bfloat16, 384, 384)])
def test_partial_gradient_requests_give_the_same_gradients_and_skip_the_rest(dtype, D, F):
    """Frozen parameters, an input that needs no gradient and a trainable gate bias: every gradient that
    is asked for equals the one of the run where everything is trainable (bit for bit: the same kernels
    run), and nothing is returned for what was not asked.  (The autograd nodes of the block's operators
    index needs_input_grad by tensor argument; linear.py:133-151 has the gate's three gradients.)"""
    T, E, K = 200, 8, 2
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True)
    p = make_params(E, D, F, dtype, seed=3, std=0.1, shared_F=F)
    p.router_logit_bias_E = torch.linspace(-0.2, 0.2, E)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, D, generator=g).to(dtype).to(DEV)
    gout = torch.randn(T, D, generator=g).to(dtype).to(DEV)

    def run(frozen=(), x_grad=True, bias_grad=False):
        block = build_block(p, spec, D, F, dtype, DEV)
        block.train()
        block.router.gate.bias.requires_grad_(bias_grad)
        named = dict(block.named_parameters())
        for name in frozen:
            named[name].requires_grad_(False)
        xin = x.clone().requires_grad_(x_grad)
        block(xin).backward(gout)
        grads = {n: q.grad for n, q in named.items()}
        grads["x"] = xin.grad
        return grads

    full = run(bias_grad=True)
    assert all(v is not None for v in full.values())
    # the gate bias gradient against the oracle's, with the bias as a leaf of the oracle's graph
    leaves = {k: getattr(p, k).clone() for k in
              ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF", "shared_gate_FD", "shared_up_FD", "shared_down_DF")}
    bias_leaf = p.router_logit_bias_E.clone().requires_grad_()
    ref, _ = R.moe_forward(x.cpu(), R.MoEParams(expert_bias_E=None, router_logit_bias_E=bias_leaf, **leaves), spec)
    ref.backward(gout.cpu())
    tol, metric = (1e-5, rel_max) if dtype == torch.float32 else (2e-2, rel_l2)
    assert full["router.gate.bias"].shape == (E,)
    assert metric(full["router.gate.bias"], bias_leaf.grad) < tol, metric(full["router.gate.bias"], bias_leaf.grad)
    cases = [
        dict(frozen=("routed_experts.inner_experts.w1_EFD",)),
        dict(frozen=("routed_experts.inner_experts.w3_EFD", "routed_experts.inner_experts.w2_EDF")),
        dict(frozen=("router.gate.weight",), bias_grad=True),
        dict(frozen=("shared_experts.up_proj.weight",), x_grad=False),
        dict(frozen=tuple(n for n in full if n not in ("x", "router.gate.bias")), x_grad=True),
        dict(x_grad=False, bias_grad=True),
    ]
    for case in cases:
        got = run(**case)
        skipped = set(case.get("frozen", ()))
        if not case.get("x_grad", True):
            skipped.add("x")
        if not case.get("bias_grad", False):
            skipped.add("router.gate.bias")
        for name, want in full.items():
            if name in skipped:
                assert got[name] is None, (case, name)
            else:
                assert got[name] is not None and torch.equal(got[name], want), (case, name)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,D,F,shared_F", [(torch.float32, 64, 96, None), (torch.bfloat16, 384, 384, None),
                                                (torch.bfloat16, 384, 384, 384)])
def test_whole_block_traces_as_one_graph_and_equals_eager(dtype, D, F, shared_F):
    """The block under torch.compile(backend="aot_eager", fullgraph=True) -- one graph, forward and
    backward through the operators' fake kernels and autograd nodes -- gives the eager step bit for bit:
    output, every gradient, and the counters the block commits.  (The reference traces its experts this
    way, tests/unit_tests/cpu/test_expert_compile_segments.py:13-40; here the whole block does.)"""
    print(f"block under torch.compile {dtype} D={D} F={F} shared={shared_F}", flush=True)
    T, E, K = 300, 8, 2
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True)
    p = make_params(E, D, F, dtype, seed=3, std=0.1, shared_F=shared_F)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, D, generator=g).to(dtype).to(DEV)
    gout = torch.randn(T, D, generator=g).to(dtype).to(DEV)

    def run(compiled):
        block = build_block(p, spec, D, F, dtype, DEV)
        block.train()
        block.overlap_shared_experts = False  # (a traced block runs on one stream: the same summation order)
        fn = torch.compile(block, backend="aot_eager", fullgraph=True) if compiled else block
        xin = x.clone().requires_grad_()
        out = fn(xin)
        out.backward(gout)
        return [out.detach(), xin.grad] + [q.grad for q in block.parameters()] + [block.tokens_per_expert_E.clone()]

    torch._dynamo.reset()
    eager, traced = run(False), run(True)
    assert len(eager) == len(traced)
    for i, (a, b) in enumerate(zip(eager, traced)):
        assert a is not None and b is not None and torch.equal(a, b), i
    assert eager[-1].sum() == T * K


@pytest.mark.gpu
@pytest.mark.parametrize("kw", [dict(dispatcher="padded", pad_multiple=128), dict(dispatcher="share", local=(2, 6)),
                                dict(load_balance_coeff=1e-3)], ids=["padded", "local-share", "expert-bias"])
def test_traced_block_with_the_other_dispatchers_and_the_expert_bias_equals_eager(kw):
    """The same one-graph trace for the padded layout, one rank's share of the experts, and a block that
    carries the load-balancing bias and its counters."""
    print(f"block under torch.compile {kw}", flush=True)
    dtype, D, F, T, E, K = torch.bfloat16, 384, 384, 300, 8, 2
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=False)
    p = make_params(E, D, F, dtype, seed=3, std=0.1)
    if kw.get("dispatcher") == "share":
        for name in ("w1_EFD", "w3_EFD", "w2_EDF"):
            setattr(p, name, getattr(p, name)[2:6].clone())
    if "load_balance_coeff" in kw:
        p.expert_bias_E = torch.linspace(-0.1, 0.1, E)
    g = torch.Generator().manual_seed(11)
    x = torch.randn(T, D, generator=g).to(dtype).to(DEV)
    gout = torch.randn(T, D, generator=g).to(dtype).to(DEV)

    def run(compiled):
        block = build_block(p, spec, D, F, dtype, DEV, **kw)
        block.train()
        fn = torch.compile(block, backend="aot_eager", fullgraph=True) if compiled else block
        xin = x.clone().requires_grad_()
        fn(xin).backward(gout)
        return [xin.grad] + [q.grad for q in block.parameters()] + [block.tokens_per_expert_E.clone()]

    torch._dynamo.reset()
    for i, (a, b) in enumerate(zip(run(False), run(True))):
        assert (a is None and b is None) or torch.equal(a, b), i


@pytest.mark.gpu
@pytest.mark.parametrize("dtype,D,F", [(torch.float32, 64, 96), (torch.bfloat16, 384, 384)])
def test_second_backward_through_a_kept_graph_and_checkpointed_recomputation(dtype, D, F):
    """The autograd nodes keep what they saved when the graph is kept: a second backward pass gives the
    same gradients again (accumulated: exactly twice the first).  Under torch.utils.checkpoint the block
    is run again inside the backward pass: the same output gradient reaches the same kernels, so input
    and weight gradients equal the plain run's bit for bit."""
    from torch.utils.checkpoint import checkpoint

    T, E, K = 150, 8, 2
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, dtype, seed=9, std=0.1, shared_F=F)
    g = torch.Generator().manual_seed(21)
    x = torch.randn(T, D, generator=g).to(dtype).to(DEV)
    gout = torch.randn(T, D, generator=g).to(dtype).to(DEV)

    def grads_of(block, xin):
        return [xin.grad.clone()] + [q.grad.clone() for q in block.parameters()]

    block = build_block(p, spec, D, F, dtype, DEV)
    block.train()
    block.overlap_shared_experts = False
    xin = x.clone().requires_grad_()
    out = block(xin)
    out.backward(gout, retain_graph=True)
    once = grads_of(block, xin)
    out.backward(gout)
    twice = grads_of(block, xin)
    for a, b in zip(once, twice):
        assert torch.equal(b.float(), 2 * a.float()) or rel_max(b.float(), 2 * a.float()) < 1e-2  # bf16 accumulation rounds

    block2 = build_block(p, spec, D, F, dtype, DEV)
    block2.train()
    block2.overlap_shared_experts = False
    xin2 = x.clone().requires_grad_()
    checkpoint(block2, xin2, use_reentrant=False).backward(gout)
    for a, b in zip(once, grads_of(block2, xin2)):
        assert torch.equal(a, b)
    # the replay stops at the last tensor the backward needs, before the block commits its counters at the
    # end of forward (layer.py:246-309 commits last for the same reason): one pass is counted.  A wrapper
    # that replays whole forwards sets the reference's context variable (models/common/aux_loss.py:42-43)
    # and has the replay skipped, below.
    assert block2.tokens_per_expert_E.sum() == T * K

    from contextlib import contextmanager, nullcontext

    from torchllmtuner_amd.moe.layer import in_checkpoint_recompute

    @contextmanager
    def replaying():
        token = in_checkpoint_recompute.set(True)
        try:
            yield
        finally:
            in_checkpoint_recompute.reset(token)

    block3 = build_block(p, spec, D, F, dtype, DEV)
    block3.train()
    block3.overlap_shared_experts = False
    xin3 = x.clone().requires_grad_()
    checkpoint(block3, xin3, use_reentrant=False, context_fn=lambda: (nullcontext(), replaying())).backward(gout)
    for a, b in zip(once, grads_of(block3, xin3)):
        assert torch.equal(a, b)
    assert block3.tokens_per_expert_E.sum() == T * K
