"""fp64 through the boundary: the reference runs its experts in fp64 on the CPU
(tests/unit_tests/cpu/test_expert_compile_segments.py:13-40) and its router converts fp64 operands
to fp32 (llmtuner/models/common/linear.py:123-125).  Row movers, combine, grouped experts and
grouped linear maps compute in fp64 here and are held to 1e-12 against the CPU oracle (the sums
run in another order); whatever passes through the fp32 router is held to the fp32 bar, 1e-5.
"""

import pytest
import torch

from oracle import moe_ref as R
from tests.helpers import build_block, make_params, rel_max

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
F64_TOL = 1e-12


@pytest.fixture(scope="module")
def ops():
    from torchllmtuner_amd import ops as _ops

    return _ops


def test_router_gate_takes_fp64_operands_and_computes_in_fp32(ops):
    print("fp64 router gate", flush=True)
    g = torch.Generator().manual_seed(0)
    T, D, E = 300, 72, 12
    x = torch.randn(T, D, generator=g, dtype=F64)
    gout = torch.randn(T, E, generator=g)
    for wdt in (torch.float32, F64):
        w = (torch.randn(E, D, generator=g) * 0.05).to(wdt)
        xr, wr = x.clone().requires_grad_(), w.clone().requires_grad_()
        ref = R.router_gate(xr, wr)
        ref.backward(gout)
        got = ops.router_gate_fwd(x.to(DEV), w.to(DEV))
        assert got.dtype == torch.float32
        assert rel_max(got, ref) < 1e-5
        dx, dw = ops.router_gate_bwd(gout.to(DEV), x.to(DEV), w.to(DEV))
        assert dx.dtype == F64 and dw.dtype == wdt
        assert rel_max(dx, xr.grad) < 1e-5 and rel_max(dw, wr.grad) < 1e-5
        # the values are fp32 values (linear.py:138-149 casts the fp32 products back)
        assert torch.equal(dx, dx.float().double())


@pytest.mark.parametrize("T,K,E,D,align,local", [(300, 4, 16, 96, 1, None), (300, 4, 16, 37, 8, None),
                                                 (513, 8, 32, 64, 1, (4, 12)), (0, 2, 4, 8, 1, None)])
def test_rows_move_and_sum_in_fp64(ops, T, K, E, D, align, local):
    print(f"fp64 rows T={T} K={K} E={E} D={D} align={align} local={local}", flush=True)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, D, generator=g, dtype=F64)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]) if T else torch.empty(0, K, dtype=torch.long)
    lo, hi = (0, E) if local is None else local
    plan = ops.permute_plan(ids.to(DEV), E, lo, hi, align)
    rows = ops.permute_rows_fwd(x.to(DEV), plan)
    assert rows.dtype == F64
    total = int(plan.total_rows.item())
    xr = x.clone().requires_grad_()
    rows_ref, _, _, _ = R.local_reorder(xr, torch.ones(T, K, dtype=F64), ids)
    counts = torch.bincount(ids.reshape(-1), minlength=E)
    rows_ref = rows_ref[int(counts[:lo].sum()): int(counts[:hi].sum())]
    _, padded_ref, _, _ = R.permute_and_pad(rows_ref, counts[lo:hi], align)
    assert total == padded_ref.shape[0]
    assert torch.equal(rows.cpu()[:total], padded_ref.detach())  # a copy: every bit
    grows = torch.randn(total, D, generator=g, dtype=F64)
    padded_ref.backward(grows)
    buf = torch.zeros(plan.row_capacity, D, dtype=F64)
    buf[:total] = grows
    dx = ops.permute_rows_bwd(buf.to(DEV), plan)
    if T:
        assert dx.dtype == F64 and rel_max(dx, xr.grad) < F64_TOL


@pytest.mark.parametrize("top_k,tokens", [(2, 64), (8, 1000), (3, 0)])
def test_combine_in_fp64(ops, top_k, tokens):
    # the reference's fp64 exactness check: tests/unit_tests/cpu/parallel/test_moe_token_dispatch.py:84-99
    print(f"fp64 combine k={top_k} T={tokens}", flush=True)
    torch.manual_seed(91)
    hidden = 100
    ids = torch.randint(0, 16, (tokens, top_k))
    values = torch.randn(tokens * top_k, hidden, dtype=F64) * 0.1
    scores = torch.rand(tokens, top_k)
    probe = torch.randn(tokens, hidden, dtype=F64)
    order = ids.flatten().argsort(stable=True)
    vr, sr = values.clone().requires_grad_(), scores.clone().requires_grad_()
    ref = R.combine(vr, order // top_k, sr.flatten()[order], values.new_empty(tokens, hidden))
    plan = ops.permute_plan(ids.to(DEV), 16)
    got = ops.combine_fwd(values.to(DEV), scores.to(DEV), plan)
    assert got.dtype == F64 and got.shape == (tokens, hidden)
    if tokens == 0:
        return
    assert rel_max(got, ref) < F64_TOL
    ref.backward(probe)
    dy, dw = ops.combine_bwd(probe.to(DEV), values.to(DEV), scores.to(DEV), plan)
    assert dy.dtype == F64 and dw.dtype == torch.float32
    assert rel_max(dy, vr.grad) < F64_TOL
    assert rel_max(dw, sr.grad) < 1e-6  # an fp64 sum rounded once to the scores' fp32


@pytest.mark.parametrize("counts,D,Fd", [((2, 0, 3), 4, 8), ((0, 5, 0), 4, 8), ((0, 0, 0), 4, 8),
                                         ((130, 1, 64, 300), 16, 32), ((100, 0, 29), 72, 40)])
def test_grouped_experts_in_fp64(ops, counts, D, Fd):
    """The counts of tests/unit_tests/cpu/test_expert_compile_segments.py:13-40 (and larger ones):
    forward and all four gradients of the fp64 experts against the oracle's fp64 loop."""
    print(f"fp64 experts {counts} D={D} F={Fd}", flush=True)
    g = torch.Generator().manual_seed(77)
    El, Rn = len(counts), sum(counts)
    x = torch.randn(Rn, D, generator=g, dtype=F64)
    ws = [torch.randn(El, Fd, D, generator=g, dtype=F64) * 0.1, torch.randn(El, Fd, D, generator=g, dtype=F64) * 0.1,
          torch.randn(El, D, Fd, generator=g, dtype=F64) * 0.1]
    gy = torch.randn(Rn, D, generator=g, dtype=F64)
    ref_in = [t.clone().requires_grad_() for t in (x, *ws)]
    ref = R.grouped_experts(ref_in[0], torch.tensor(counts), *ref_in[1:])
    if Rn:
        ref.backward(gy)
    else:
        ref.sum().backward()
    plan = ops.segments_from_counts(torch.tensor(counts, dtype=torch.int32, device=DEV), Rn)
    xd, w1, w3, w2 = (t.to(DEV) for t in (x, *ws))
    y, gate, up, h = ops.grouped_swiglu_fwd(xd, w1, w3, w2, plan)
    assert y.dtype == F64
    if Rn:
        assert rel_max(y, ref) < F64_TOL
    grads = ops.grouped_swiglu_bwd(gy.to(DEV), xd, w1, w3, w2, gate, up, h, plan)
    for name, got, want in zip(("drows", "dw1", "dw3", "dw2"), grads, (t.grad for t in ref_in)):
        assert got.dtype == F64 and got.shape == want.shape, name
        if want.numel() == 0 or want.abs().max() == 0:
            assert got.numel() == 0 or got.abs().max() == 0, name
        else:
            assert rel_max(got, want) < F64_TOL, f"{name} {rel_max(got, want)}"


@pytest.mark.parametrize("activation", ["swiglu", "situ"])
def test_grouped_experts_module_in_fp64_with_autograd(ops, activation):
    from torchllmtuner_amd import moe

    print(f"fp64 experts module {activation}", flush=True)
    g = torch.Generator().manual_seed(3)
    counts, D, Fd = (7, 0, 70, 3), 24, 40
    El, Rn = len(counts), sum(counts)
    x = torch.randn(Rn, D, generator=g, dtype=F64)
    ws = [torch.randn(El, Fd, D, generator=g, dtype=F64) * 0.1, torch.randn(El, Fd, D, generator=g, dtype=F64) * 0.1,
          torch.randn(El, D, Fd, generator=g, dtype=F64) * 0.1]
    gy = torch.randn(Rn, D, generator=g, dtype=F64)
    ref_in = [t.clone().requires_grad_() for t in (x, *ws)]
    act = None if activation == "swiglu" else (lambda a, b: R.situ_glu(a, b, 1.5, 0.8))
    R.grouped_experts(ref_in[0], torch.tensor(counts), *ref_in[1:], act).backward(gy)
    fn = None if activation == "swiglu" else moe.SituGLU(1.5, 0.8)
    experts = moe.GroupedExperts(D, Fd, El, activation_fn=fn).to(DEV).double()
    with torch.no_grad():
        for prm, t in zip((experts.w1_EFD, experts.w3_EFD, experts.w2_EDF), ws):
            prm.copy_(t)
    xd = x.to(DEV).requires_grad_()
    experts(xd, torch.tensor(counts, device=DEV)).backward(gy.to(DEV))
    # SituGLU computes in fp32 by definition (activation.py:58-64): that case is held to the fp32 bar
    tol = F64_TOL if activation == "swiglu" else 1e-5
    for name, got, want in (("dx", xd.grad, ref_in[0].grad), ("dw1", experts.w1_EFD.grad, ref_in[1].grad),
                            ("dw3", experts.w3_EFD.grad, ref_in[2].grad), ("dw2", experts.w2_EDF.grad, ref_in[3].grad)):
        assert got.dtype == F64 and rel_max(got, want) < tol, f"{name} {rel_max(got, want)}"


@pytest.mark.parametrize("with_fp64_router", [False, True])
def test_whole_block_in_fp64(with_fp64_router):
    """The C1-sized block with every parameter and the tokens in fp64.  Routing runs in fp32 on
    both sides, so the block is held to the fp32 bar; the routing decision must be the oracle's."""
    print(f"fp64 block router_fp64={with_fp64_router}", flush=True)
    T, D, E, K, F = 512, 64, 8, 2, 96
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=True)
    p = make_params(E, D, F, F64, seed=0, shared_F=48)
    if with_fp64_router:
        p.router_w_ED = p.router_w_ED.double()
    x = torch.randn(2, T // 2, D, generator=torch.Generator().manual_seed(0), dtype=F64)
    gout = torch.randn(2, T // 2, D, generator=torch.Generator().manual_seed(1), dtype=F64)
    leaves = {k: getattr(p, k).clone().requires_grad_() for k in
              ("router_w_ED", "w1_EFD", "w3_EFD", "w2_EDF", "shared_gate_FD", "shared_up_FD", "shared_down_DF")}
    xr = x.clone().requires_grad_()
    ref, aux = R.moe_forward(xr, R.MoEParams(**leaves), spec)
    ref.backward(gout)
    block = build_block(p, spec, D, F, F64, DEV)
    if with_fp64_router:
        block.router.gate.double()
        with torch.no_grad():
            block.router.gate.weight.copy_(p.router_w_ED)
    xd = x.to(DEV).requires_grad_()
    out = block(xd)
    assert out.dtype == F64 and out.shape == x.shape
    out.backward(gout.to(DEV))
    _, ids = block.router.route(x.reshape(-1, D).to(DEV))
    assert torch.equal(ids.cpu(), aux["ids_TK"])
    ie, sh = block.routed_experts.inner_experts, block.shared_experts
    got = {"out": out, "dx": xd.grad, "router_w_ED": block.router.gate.weight.grad, "w1_EFD": ie.w1_EFD.grad,
           "w3_EFD": ie.w3_EFD.grad, "w2_EDF": ie.w2_EDF.grad, "shared_gate_FD": sh.gate_proj.weight.grad,
           "shared_up_FD": sh.up_proj.weight.grad, "shared_down_DF": sh.down_proj.weight.grad}
    want = {"out": ref, "dx": xr.grad, **{k: v.grad for k, v in leaves.items()}}
    for k in want:
        assert got[k].dtype == want[k].dtype, k
        assert rel_max(got[k], want[k]) < 1e-5, f"{k}: {rel_max(got[k], want[k])}"
    # the shared expert sees no routing: its weight gradients carry the full fp64 precision
    # up to the output gradient they are fed, which is exact
    assert rel_max(got["shared_down_DF"], want["shared_down_DF"]) < F64_TOL


def test_kernels_without_an_fp64_form_say_so(ops):
    print("fp64 refusals", flush=True)
    x = torch.randn(4, 8, device=DEV, dtype=F64)
    with pytest.raises(TypeError, match="float32 and bfloat16, got torch.float64"):
        ops.rms_norm_fwd(x, torch.ones(8, device=DEV, dtype=F64), 1e-6)


# ---- derivative checks by finite differences: independent of the oracle ------------------------------
# torch.autograd.gradcheck perturbs every input element (central differences in fp64) and compares the
# numerical Jacobian with the one the backward kernels give; it also re-runs the backward for
# determinism and feeds undefined output gradients.  Sizes are tiny: one forward per perturbation.
def _gradcheck(fn, inputs):
    return torch.autograd.gradcheck(fn, inputs, eps=1e-6, atol=1e-8, rtol=1e-6, nondet_tol=0.0)


@pytest.mark.parametrize("counts", [(3, 0, 4), (1, 1, 1, 1), (0, 6)])
def test_grouped_experts_backward_is_the_derivative_of_the_forward(ops, counts):
    print(f"fp64 gradcheck experts {counts}", flush=True)
    g = torch.Generator().manual_seed(5)
    El, Rn, D, Fd = len(counts), sum(counts), 4, 6
    plan = ops.segments_from_counts(torch.tensor(counts, dtype=torch.int32, device=DEV), Rn)
    x = torch.randn(Rn, D, generator=g, dtype=F64).to(DEV).requires_grad_()
    w1, w3 = (torch.randn(El, Fd, D, generator=g, dtype=F64).mul(0.5).to(DEV).requires_grad_() for _ in range(2))
    w2 = torch.randn(El, D, Fd, generator=g, dtype=F64).mul(0.5).to(DEV).requires_grad_()
    assert _gradcheck(lambda a, b, c, d: ops.grouped_swiglu_fwd(a, b, c, d, plan)[0], (x, w1, w3, w2))


def test_grouped_linear_backward_is_the_derivative_of_the_forward(ops):
    print("fp64 gradcheck grouped linear", flush=True)
    g = torch.Generator().manual_seed(6)
    counts, I, O = (2, 0, 5, 1), 5, 3
    plan = ops.segments_from_counts(torch.tensor(counts, dtype=torch.int32, device=DEV), sum(counts))
    x = torch.randn(sum(counts), I, generator=g, dtype=F64).to(DEV).requires_grad_()
    w = torch.randn(len(counts), O, I, generator=g, dtype=F64).to(DEV).requires_grad_()
    assert _gradcheck(lambda a, b: ops.grouped_linear(a, b, plan), (x, w))


def test_row_movers_and_combine_backward_are_the_derivatives_of_the_forward(ops):
    print("fp64 gradcheck movers", flush=True)
    g = torch.Generator().manual_seed(7)
    T, K, E, D = 9, 3, 5, 4
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    plan = ops.permute_plan(ids.to(DEV), E)
    x = torch.randn(T, D, generator=g, dtype=F64).to(DEV).requires_grad_()
    assert _gradcheck(lambda a: ops.permute_rows_fwd(a, plan), (x,))
    y = torch.randn(T * K, D, generator=g, dtype=F64).to(DEV).requires_grad_()
    scores = torch.rand(T, K, generator=g).to(DEV)
    assert _gradcheck(lambda a: ops.combine_fwd(a, scores, plan), (y,))


def test_staged_routed_path_backward_is_the_derivative_of_the_forward(ops):
    """Row scatter + experts + combine as the one operator the block uses where no folded kernel
    applies, differentiated in the tokens and the three weight stacks."""
    print("fp64 gradcheck staged path", flush=True)
    g = torch.Generator().manual_seed(8)
    T, K, E, D, Fd = 7, 2, 4, 4, 6
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    plan = ops.permute_plan(ids.to(DEV), E)
    scores = torch.rand(T, K, generator=g).to(DEV)
    x = torch.randn(T, D, generator=g, dtype=F64).to(DEV).requires_grad_()
    w1, w3 = (torch.randn(E, Fd, D, generator=g, dtype=F64).mul(0.5).to(DEV).requires_grad_() for _ in range(2))
    w2 = torch.randn(E, D, Fd, generator=g, dtype=F64).mul(0.5).to(DEV).requires_grad_()
    assert _gradcheck(lambda a, b, c, d: ops.rows_experts_combine(a, scores, b, c, d, plan, True), (x, w1, w3, w2))
