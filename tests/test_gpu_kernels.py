"""GPU parity of every kernel, called through the C ABI (torchllmtuner_amd.ops),
against the CPU oracle on identical seeded inputs.

Bars: routing ids, counts and permutation order bit-exact -- on EVERY token whose oracle
scores do not tie exactly where the choice is the plain top-k of the scores (the kernel then
selects on the logits, which no exp() implementation can reorder), and on every token
outside the few-ulp near-tie set (helpers.stable_tokens), with the number of differing
tokens printed and bounded, where a bias or group scores enter the choice; fp32 values
within 1e-5 relative; bf16 values within 2e-2 relative L2.
"""

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_ref as R
from tests.helpers import exact_score_ties, note, rel_l2, rel_max, stable_tokens

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
FP32_TOL = 1e-5
BF16_TOL = 2e-2


@pytest.fixture(scope="module")
def ops():
    from torchllmtuner_amd import ops as _ops

    return _ops


# ---------------------------------------------------------------- router gate
@pytest.mark.parametrize("T,D,E,xdt", [(3, 8, 4, torch.float32), (512, 256, 8, torch.float32),
                                       (1000, 320, 72, torch.bfloat16), (0, 16, 4, torch.float32),
                                       # bf16 tokens, D and E multiples of 64: the three-piece bf16 MFMA path
                                       (1000, 320, 64, torch.bfloat16), (2048, 2048, 128, torch.bfloat16),
                                       (77, 192, 192, torch.bfloat16), (8192, 128, 256, torch.bfloat16),
                                       # 128-token tiles: ragged T and E, with and without a split contraction
                                       (1100, 448, 192, torch.bfloat16), (1100, 1024, 192, torch.bfloat16)])
def test_router_gate_fwd_bwd(ops, T, D, E, xdt):
    print(f"router_gate T={T} D={D} E={E} {xdt}", flush=True)
    g = torch.Generator().manual_seed(0)
    x = torch.randn(T, D, generator=g).to(xdt)
    w = torch.randn(E, D, generator=g) * 0.05
    b = torch.randn(E, generator=g)
    gout = torch.randn(T, E, generator=g)
    xr, wr = x.clone().requires_grad_(), w.clone().requires_grad_()
    ref = R.router_gate(xr, wr, b)
    got = ops.router_gate_fwd(x.to(DEV), w.to(DEV), b.to(DEV))
    assert got.dtype == torch.float32 and got.shape == (T, E)
    if T == 0:
        return
    assert rel_max(got, ref) < FP32_TOL
    ref.backward(gout)
    dx, dw = ops.router_gate_bwd(gout.to(DEV), x.to(DEV), w.to(DEV))
    assert dx.dtype == xdt and dw.dtype == torch.float32
    assert rel_max(dx, xr.grad) < (FP32_TOL if xdt == torch.float32 else 1e-2)
    assert rel_max(dw, wr.grad) < FP32_TOL


# ---------------------------------------------------------------- router select
SELECT_CASES = [
    dict(T=512, E=8, K=2, score_func="softmax", route_norm=True),
    dict(T=2048, E=128, K=8, score_func="softmax", route_norm=True),
    dict(T=1024, E=256, K=8, score_func="sigmoid", route_norm=True, route_scale=2.5,
         num_expert_groups=8, num_limited_groups=4, bias=True),
    dict(T=300, E=64, K=6, score_func="sigmoid", bias=True),
    # the 16-lanes-per-token kernel at its other widths and its K limits
    dict(T=333, E=256, K=16, score_func="sqrtsoftplus", route_norm=True, bias=True),
    dict(T=77, E=128, K=1, score_func="softmax"),
    dict(T=100, E=256, K=17, score_func="softmax", route_norm=True),
    dict(T=300, E=24, K=3, score_func="sqrtsoftplus", route_norm=True, route_scale=0.5),
    dict(T=257, E=320, K=5, score_func="softmax", num_expert_groups=5, num_limited_groups=2),
    # groups of 2, 16, 24 (no aligned lane run), 128 (two registers per lane) experts
    dict(T=300, E=16, K=3, score_func="softmax", num_expert_groups=8, num_limited_groups=2),
    dict(T=300, E=128, K=6, score_func="sigmoid", route_norm=True, num_expert_groups=8, num_limited_groups=3, bias=True),
    dict(T=300, E=96, K=4, score_func="sigmoid", num_expert_groups=4, num_limited_groups=2, bias=True),
    dict(T=300, E=256, K=8, score_func="softmax", route_norm=True, num_expert_groups=2, num_limited_groups=1),
    dict(T=300, E=512, K=8, score_func="sigmoid", num_expert_groups=4, num_limited_groups=2, bias=True),
    # one lane per group and one group in all, in the 16-lanes-per-token kernel
    dict(T=300, E=64, K=4, score_func="sigmoid", route_norm=True, num_expert_groups=16, num_limited_groups=4, bias=True),
    dict(T=300, E=128, K=5, score_func="softmax", num_expert_groups=1, num_limited_groups=1),
    dict(T=10, E=4, K=2, score_func="sigmoid", fixed_router=True, route_scale=7.0),
    dict(T=10, E=4, K=2, score_func="sigmoid", debug_force_load_balance=True, route_norm=True, route_scale=2.0),
]


@pytest.mark.parametrize("case", SELECT_CASES,
                         ids=lambda c: f"E{c['E']}K{c['K']}{c['score_func']}" + (f"G{c['num_expert_groups']}" if "num_expert_groups" in c else ""))
def test_router_select_fwd_bwd(ops, case):
    print(f"router_select {case}", flush=True)
    c = dict(case)
    T, E, K = c.pop("T"), c.pop("E"), c.pop("K")
    use_bias = c.pop("bias", False)
    spec = R.RouterSpec(E, K, **c)
    g = torch.Generator().manual_seed(7)
    logits = torch.randn(T, E, generator=g) * 1.5
    bias = (torch.rand(E, generator=g) * 0.2 - 0.1) if use_bias else None
    lr = logits.clone().requires_grad_()
    w_ref, ids_ref, _ = R.route(lr, spec, bias)
    mode = 1 if spec.fixed_router else (2 if spec.debug_force_load_balance else 0)
    w, ids, scores, rmap = ops.router_select_fwd(
        logits.to(DEV), None if bias is None else bias.to(DEV), K, spec.score_func, spec.route_norm,
        spec.route_scale, spec.num_expert_groups or 0, spec.num_limited_groups or 0, mode, True, True)
    assert ids.dtype == torch.int64 and rmap.dtype == torch.bool
    # the routing map is the one-hot of the kernel's own ids (routing.py:320-324)
    assert torch.equal(rmap.cpu(), torch.zeros(T, E, dtype=torch.bool).scatter_(-1, ids.cpu(), True))
    differ = ~(ids.cpu() == ids_ref).all(-1)
    if mode:
        assert not differ.any()
        ok = torch.ones(T, dtype=torch.bool)
    elif bias is None and not spec.num_expert_groups:
        # plain top-k of the scores: bit-exact on every token whose scores do not tie exactly
        # (where the reference's own torch.topk is free to pick either)
        tied = exact_score_ties(logits, spec)
        note(f"select {spec.score_func} E={E} K={K}: {int(tied.sum())} of {T} tokens have an exact score tie among "
             f"the top {K + 1}; {int(differ.sum())} tokens differ from the oracle")
        assert int(tied.sum()) <= max(1, T // 100)
        assert not differ[~tied].any(), "routing ids differ although the logits are identical and no score ties"
        ok = ~tied
    else:
        # a bias or group scores enter the choice: two correct exp() implementations may flip a
        # token whose decision hangs on the last ulps; every difference must be such a token
        ok = stable_tokens(logits, spec, bias)
        note(f"select {spec.score_func} E={E} K={K} (bias / groups): {int((~ok).sum())} of {T} tokens are near "
             f"ties; {int(differ.sum())} tokens differ from the oracle")
        assert ok.float().mean() > 0.98, "too many near-tie tokens for a meaningful check"
        assert not differ[ok].any(), "routing ids differ on tokens that are not near ties"
        assert int(differ.sum()) <= int((~ok).sum())
    assert rel_max(scores, R.score(logits, spec.score_func)) < FP32_TOL
    assert rel_max(w.cpu()[~differ], w_ref[~differ]) < FP32_TOL
    # backward given the oracle's ids (same inputs on both sides)
    gw = torch.randn(T, K, generator=g)
    if not spec.fixed_router:
        w_ref.backward(gw)
        dl = ops.router_select_bwd(logits.to(DEV), ids_ref.to(DEV), gw.to(DEV), None, spec.score_func,
                                   spec.route_norm, spec.route_scale, mode)
        assert rel_max(dl, lr.grad) < 2e-5
    # dense score gradient path (aux-loss hook)
    lr2 = logits.clone().requires_grad_()
    gs = torch.randn(T, E, generator=g)
    R.score(lr2, spec.score_func).backward(gs)
    dl2 = ops.router_select_bwd(logits.to(DEV), ids_ref.to(DEV), None, gs.to(DEV), spec.score_func,
                                spec.route_norm, spec.route_scale, mode)
    assert rel_max(dl2, lr2.grad) < 2e-5


def test_router_select_exact_ties_go_to_lower_index(ops):
    logits = torch.zeros(5, 16)
    logits[1, 3] = logits[1, 9] = 1.0
    for fn in ("softmax", "sigmoid"):
        w, ids, _ = ops.router_select_fwd(logits.to(DEV), None, 4, fn, False, 1.0)
        assert ids[0].tolist() == [0, 1, 2, 3]
        assert ids[1].tolist() == [3, 9, 0, 1]
    # the same rule at the widths served by the 16-lanes-per-token kernel; the routing map and the
    # cutoff (the best score left) follow the same choice
    for E in (64, 128, 256):
        logits = torch.zeros(19, E)
        logits[1, 3] = logits[1, E - 7] = 1.0
        logits[2, E - 1] = 2.0
        for fn in ("softmax", "sigmoid", "sqrtsoftplus"):
            w, ids, _, rmap = ops.router_select_fwd(logits.to(DEV), None, 4, fn, True, 1.0, 0, 0, 0, False, True)
            assert ids[0].tolist() == [0, 1, 2, 3] and ids[18].tolist() == [0, 1, 2, 3]
            assert ids[1].tolist() == [3, E - 7, 0, 1]
            assert ids[2].tolist() == [E - 1, 0, 1, 2]
            assert torch.equal(rmap.cpu(), torch.zeros(19, E, dtype=torch.bool).scatter_(-1, ids.cpu(), True))
            assert torch.allclose(w.sum(-1).cpu(), torch.ones(19), atol=1e-6)
    # grouped known answer: tests/unit_tests/cpu/models/test_models_common.py:157-165
    s = torch.tensor([[0.80, 0.70, 0.00, 0.00, 0.90, 0.20, 0.00, 0.00]])
    lg = torch.log(s.clamp_min(1e-6) / (1 - s).clamp_min(1e-6))  # sigmoid^-1
    _, ids, _ = ops.router_select_fwd(lg.to(DEV), None, 2, "sigmoid", False, 1.0, 2, 1)
    assert ids.tolist() == [[0, 1]]


@pytest.mark.parametrize("E,K,groups", [(64, 6, 0), (128, 8, 0), (256, 8, 0), (256, 8, 8), (128, 4, 4)])
def test_both_select_kernels_make_the_same_choice(ops, E, K, groups):
    """The 16-lanes-per-token kernel (16-byte aligned logits, E = 64 / 128 / 256) and the
    wavefront-per-token kernel (any alignment) choose the same experts on every token: their
    comparisons differ in order only, and (larger value, lower index) is a total order.  With
    sigmoid scores nothing is summed before the choice, so weights and scores agree bit for bit
    as well; with softmax the choice is made on the logits and the scores differ by rounding."""
    print(f"select kernels agree E={E} K={K} groups={groups}", flush=True)
    T = 1000
    g = torch.Generator().manual_seed(E + K)
    aligned = torch.randn(T, E, generator=g).to(DEV)
    flat = torch.empty(T * E + 4, device=DEV)
    flat[1:1 + T * E] = aligned.view(-1)
    shifted = flat[1:1 + T * E].view(T, E)  # the same values 4 bytes into an allocation
    assert aligned.data_ptr() % 16 == 0 and shifted.data_ptr() % 16 == 4
    bias = (torch.rand(E, generator=g) * 0.2 - 0.1).to(DEV)
    limited = max(1, groups // 2)
    for fn, b in (("sigmoid", bias), ("sigmoid", None), ("softmax", None), ("sqrtsoftplus", bias)):
        if fn == "softmax" and groups:
            continue  # the scores, summed in a different order, enter the group choice there
        ref = ops.router_select_fwd(shifted, b, K, fn, True, 2.0, groups, limited, 0, True, True)
        out = ops.router_select_fwd(aligned, b, K, fn, True, 2.0, groups, limited, 0, True, True)
        assert torch.equal(out[1], ref[1]), f"{fn}: the two kernels chose different experts"
        assert torch.equal(out[3], ref[3])
        if fn != "softmax":
            assert torch.equal(out[0], ref[0]) and torch.equal(out[2], ref[2])
        else:
            assert rel_max(out[0], ref[0]) < 1e-6 and rel_max(out[2], ref[2]) < 1e-6


# ---------------------------------------------------------------- permutation plan
@pytest.mark.parametrize("T,K,E,align,local", [
    (3, 2, 3, 1, None), (6, 2, 4, 4, None), (700, 8, 128, 1, None), (700, 8, 128, 128, None),
    (5000, 8, 256, 1, (0, 32)), (5000, 6, 64, 16, (8, 24)), (0, 2, 4, 1, None), (1, 1, 1, 1, None),
    (8192, 8, 128, 1, None),
])
def test_permute_plan_is_the_stable_argsort(ops, T, K, E, align, local):
    print(f"plan T={T} K={K} E={E} align={align} local={local}", flush=True)
    g = torch.Generator().manual_seed(11)
    ids = torch.randint(0, E, (T, K), generator=g)  # duplicates inside a token allowed
    lo, hi = (0, E) if local is None else local
    plan = ops.permute_plan(ids.to(DEV), E, lo, hi, align)
    counts = torch.bincount(ids.reshape(-1), minlength=E)
    assert torch.equal(plan.counts_E.cpu().long(), counts)
    perm = torch.argsort(ids.reshape(-1), stable=True)
    start = int(counts[:lo].sum()); stop = int(counts[:hi].sum())
    local_perm = perm[start:stop]
    lc = counts[lo:hi]
    padded = lc + (-lc % align)
    seg_off = torch.cat([torch.zeros(1, dtype=torch.long), padded.cumsum(0)])
    assert torch.equal(plan.seg_offsets.cpu().long(), seg_off)
    assert torch.equal(plan.seg_counts.cpu().long(), lc)
    # experts by descending count, ties to the lower index (what the weight-gradient walk reads)
    assert plan.expert_order.cpu().tolist() == sorted(range(hi - lo), key=lambda j: (-int(lc[j]), j))
    total = int(seg_off[-1])
    # expected slot_of_row: each segment's slots then -1 padding
    exp = torch.full((plan.row_capacity,), -1, dtype=torch.long)
    pos = 0
    for j in range(hi - lo):
        c = int(lc[j]); o = int(seg_off[j])
        exp[o:o + c] = local_perm[pos:pos + c]; pos += c
    assert torch.equal(plan.slot_of_row.cpu().long(), exp)
    row_of_slot = plan.row_of_slot.cpu().long()
    exp_r = torch.full((T * K,), -1, dtype=torch.long)
    valid = exp >= 0
    exp_r[exp[valid]] = torch.nonzero(valid).squeeze(-1)
    assert torch.equal(row_of_slot, exp_r)
    # tile list covers exactly the real rows
    nt = int(plan.num_tiles.item()); tm = plan.tile_m
    te, tr = plan.tile_expert.cpu()[:nt].long(), plan.tile_row0.cpu()[:nt].long()
    def tile_rows(c):  # an expert's tiles are equally tall, to a multiple of 16 rows
        n = (c + tm - 1) // tm
        return tm if n <= 1 else (-(-c // n) + 15) // 16 * 16
    exp_tiles = [(j, int(seg_off[j]) + i * tile_rows(int(lc[j]))) for j in range(hi - lo)
                 for i in range((int(lc[j]) + tm - 1) // tm)]
    assert list(zip(te.tolist(), tr.tolist())) == exp_tiles
    assert total <= plan.row_capacity


def test_permute_rows_known_answer_and_duplicate_backward(ops):
    # tests/unit_tests/cpu/kernel/test_kernel_contracts.py:114-127
    x = torch.arange(12, dtype=torch.float32).reshape(3, 4)
    experts = torch.tensor([[2, 0], [0, 0], [2, 1]])
    plan = ops.permute_plan(experts.to(DEV), 3)
    rows = ops.permute_rows_fwd(x.to(DEV), plan)
    assert torch.equal(rows.cpu(), x[[0, 1, 1, 2, 0, 2]])
    wts = torch.arange(1, 25, dtype=torch.float32).reshape(6, 4)
    dx = ops.permute_rows_bwd(wts.to(DEV), plan)
    want = torch.stack([wts[0] + wts[4], wts[1] + wts[2], wts[3] + wts[5]])
    assert torch.equal(dx.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,K,E,D,align,local", [(300, 4, 16, 96, 1, None), (300, 4, 16, 100, 8, None),
                                                 (513, 8, 32, 256, 1, (4, 12)), (0, 2, 4, 8, 1, None)])
def test_permute_rows_fwd_bwd_match_oracle(ops, dtype, T, K, E, D, align, local):
    print(f"rows {dtype} T={T} K={K} E={E} D={D} align={align} local={local}", flush=True)
    g = torch.Generator().manual_seed(5)
    x = torch.randn(T, D, generator=g).to(dtype)
    sc = torch.rand(T, K, generator=g)
    # distinct experts per token, like a real top-k
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]) if T else torch.empty(0, K, dtype=torch.long)
    lo, hi = (0, E) if local is None else local
    plan = ops.permute_plan(ids.to(DEV), E, lo, hi, align)
    rows = ops.permute_rows_fwd(x.to(DEV), plan)
    total = int(plan.total_rows.item())
    xr = x.clone().float().requires_grad_()
    rows_ref, tok, _, _ = R.local_reorder(xr, sc, ids)
    counts = torch.bincount(ids.reshape(-1), minlength=E)
    start, stop = int(counts[:lo].sum()), int(counts[:hi].sum())
    rows_ref = rows_ref[start:stop]
    _, padded_ref, pidx, _ = R.permute_and_pad(rows_ref, counts[lo:hi], align)
    assert total == padded_ref.shape[0]
    assert torch.equal(rows.cpu()[:total].float(), padded_ref.detach().to(dtype).float())
    grows = torch.randn(total, D, generator=g).to(dtype)
    padded_ref.backward(grows.float())
    buf = torch.zeros(plan.row_capacity, D, dtype=dtype)
    buf[:total] = grows
    dx = ops.permute_rows_bwd(buf.to(DEV), plan)
    tol = FP32_TOL if dtype == torch.float32 else 1e-2
    if T:
        assert rel_max(dx, xr.grad) < tol


# ---------------------------------------------------------------- combine
def test_combine_literals(ops):
    # tests/unit_tests/cpu/models/test_qwen_operator_contracts.py:54-68
    tokens = torch.tensor([[1.0, 3.0], [5.0, 7.0], [11.0, 13.0]])
    experts = torch.tensor([[2, 0], [1, 2], [0, 1]])
    scores = torch.tensor([[0.1, 0.9], [0.2, 0.8], [0.7, 0.3]])
    plan = ops.permute_plan(experts.to(DEV), 3)
    rows = ops.permute_rows_fwd(tokens.to(DEV), plan)
    gains = (experts.reshape(-1)[plan.slot_of_row.cpu().long()] + 1).unsqueeze(1).float()
    out = ops.combine_fwd(rows * gains.to(DEV), scores.to(DEV), plan, round_terms=False)
    want = tokens * (scores * (experts + 1)).sum(1, keepdim=True)
    torch.testing.assert_close(out.cpu(), want)
    dy, dw = ops.combine_bwd(torch.ones(3, 2, device=DEV), rows * gains.to(DEV), scores.to(DEV), plan)
    # d out.sum / d score[t,k] = sum_d tokens[t,d] * (expert+1)
    torch.testing.assert_close(dw.cpu(), tokens.sum(1, keepdim=True) * (experts + 1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("top_k", [2, 8])
@pytest.mark.parametrize("tokens", [0, 64, 1000])
@pytest.mark.parametrize("fp32acc", [False, True])
def test_combine_matches_oracle(ops, dtype, top_k, tokens, fp32acc):
    # mirrors tests/integration_tests/routed_combine_equivalence.py:22-81
    print(f"combine {dtype} k={top_k} T={tokens} fp32acc={fp32acc}", flush=True)
    torch.manual_seed(91)
    hidden = 160
    ids = torch.randint(0, 16, (tokens, top_k))
    values = (torch.randn(tokens * top_k, hidden) * 0.1).to(dtype)
    scores = torch.rand(tokens, top_k)
    probe = torch.randn(tokens, hidden).to(dtype)
    order = ids.flatten().argsort(stable=True)
    vr, sr = values.clone().requires_grad_(), scores.clone().requires_grad_()
    ref = R.combine(vr, order // top_k, sr.flatten()[order], values.new_empty(tokens, hidden), fp32acc)
    plan = ops.permute_plan(ids.to(DEV), 16)
    got = ops.combine_fwd(values.to(DEV), scores.to(DEV), plan, round_terms=not fp32acc)
    if tokens == 0:
        assert got.shape == (0, hidden)
        return
    tol = 2e-3 if dtype == torch.bfloat16 else 2e-6
    torch.testing.assert_close(got.cpu().float(), ref.detach().float(), atol=tol, rtol=0)
    ref.backward(probe)
    dy, dw = ops.combine_bwd(probe.to(DEV), values.to(DEV), scores.to(DEV), plan)
    torch.testing.assert_close(dy.cpu().float(), vr.grad.float(), atol=tol, rtol=0)
    torch.testing.assert_close(dw.cpu(), sr.grad, atol=2e-3 if dtype == torch.bfloat16 else 2e-5, rtol=1e-5)


# ---------------------------------------------------------------- grouped experts
def _experts_case(ops, dtype, counts, D, Fd, std=0.1, seed=0):
    g = torch.Generator().manual_seed(seed)
    El = len(counts)
    Rn = sum(counts)
    x = torch.randn(Rn, D, generator=g).to(dtype)
    w1 = (torch.randn(El, Fd, D, generator=g) * std).to(dtype)
    w3 = (torch.randn(El, Fd, D, generator=g) * std).to(dtype)
    w2 = (torch.randn(El, D, Fd, generator=g) * std).to(dtype)
    gy = torch.randn(Rn, D, generator=g).to(dtype)
    ref_in = [t.clone().requires_grad_() for t in (x, w1, w3, w2)]
    ref = R.grouped_experts(ref_in[0], torch.tensor(counts), *ref_in[1:])
    plan = ops.segments_from_counts(torch.tensor(counts, dtype=torch.int32, device=DEV), Rn)
    assert plan.expert_order.cpu().tolist() == sorted(range(El), key=lambda j: (-counts[j], j))
    dx_, dw1_, dw3_, dw2_ = (t.to(DEV) for t in (x, w1, w3, w2))
    y, gate, up, h = ops.grouped_swiglu_fwd(dx_, dw1_, dw3_, dw2_, plan)
    tol = FP32_TOL if dtype == torch.float32 else BF16_TOL
    metric = rel_max if dtype == torch.float32 else rel_l2
    if Rn:
        assert metric(y, ref) < tol, f"forward {metric(y, ref)}"
        ref.backward(gy)
    else:
        ref.sum().backward()
    drows, dw1, dw3, dw2 = ops.grouped_swiglu_bwd(gy.to(DEV), dx_, dw1_, dw3_, dw2_, gate, up, h, plan)
    for name, got, want in (("drows", drows, ref_in[0].grad), ("dw1", dw1, ref_in[1].grad),
                            ("dw3", dw3, ref_in[2].grad), ("dw2", dw2, ref_in[3].grad)):
        if want.numel() == 0 or want.abs().max() == 0:
            assert got.shape == want.shape and (got.numel() == 0 or got.abs().max() == 0), name
        else:
            assert metric(got, want) < tol, f"{name} {metric(got, want)}"


@pytest.mark.parametrize("counts", [(5, 6, 4, 7), (2, 0, 3), (0, 5, 0), (0, 0, 0), (130, 1, 64, 300)])
def test_grouped_experts_fp32(ops, counts):
    print(f"experts fp32 {counts}", flush=True)
    _experts_case(ops, torch.float32, counts, 16 if len(counts) == 4 else 4, 32 if len(counts) == 4 else 8)


@pytest.mark.parametrize("counts,D,Fd", [((5, 6, 4, 7), 16, 32), ((100, 0, 29), 72, 40)])
def test_grouped_experts_bf16_generic_shapes(ops, counts, D, Fd):
    print(f"experts bf16 generic {counts} D={D} F={Fd}", flush=True)
    _experts_case(ops, torch.bfloat16, counts, D, Fd)


@pytest.mark.parametrize("counts,D,Fd", [
    ((128, 128), 64, 64), ((5, 6, 4, 7), 128, 64), ((200, 0, 129, 1, 300), 256, 192),
    ((0, 0, 0), 64, 128), ((513, 77), 512, 320), ((1000,), 256, 768),
    ((200, 0, 129), 384, 768), ((131, 260), 768, 384),
    # one segment (a dense layer run through the grouped kernels): ragged and whole last tiles
    ((1000,), 384, 512), ((512,), 512, 384), ((3,), 384, 384),
    # more experts than XCDs with a skewed, tie-laden histogram: the weight-gradient walk by
    # descending count must still visit every expert's every tile exactly once
    ((300, 0, 5, 700, 1, 64, 65, 0, 128, 129, 2, 5, 4, 250, 0, 90, 17, 33, 640), 384, 512),
])
def test_grouped_experts_bf16_mfma(ops, counts, D, Fd):
    print(f"experts bf16 mfma {counts} D={D} F={Fd}", flush=True)
    _experts_case(ops, torch.bfloat16, counts, D, Fd, std=0.05)


# ---------------------------------------------------------------- one grouped linear map
def _linear_case(ops, dtype, counts, I, O, seed=0, extra_rows=0):
    """y[segment e] = x[segment e] . w[e]^T and both gradients, against per-segment fp32 matrix
    products of the same inputs (experts.py:272-285's loop, written out here)."""
    g = torch.Generator().manual_seed(seed)
    El, Rn = len(counts), sum(counts) + extra_rows
    x = torch.randn(Rn, I, generator=g).to(dtype)
    w = (torch.randn(El, O, I, generator=g) * 0.1).to(dtype)
    gy = torch.randn(Rn, O, generator=g).to(dtype)
    covered = sum(counts)
    xs, gs = x[:covered].float().split(counts), gy[:covered].float().split(counts)
    want_y = torch.cat([xs[e] @ w[e].float().T for e in range(El)]) if covered else torch.zeros(0, O)
    want_dx = torch.cat([gs[e] @ w[e].float() for e in range(El)]) if covered else torch.zeros(0, I)
    want_dw = torch.stack([gs[e].T @ xs[e] for e in range(El)])
    plan = ops.segments_from_counts(torch.tensor(counts, dtype=torch.int32, device=DEV), Rn)
    xd, wd = x.to(DEV).requires_grad_(), w.to(DEV).requires_grad_()
    junk = torch.full((Rn + 1, max(I, O)), float("nan"), device=DEV, dtype=dtype)  # poison the free blocks
    del junk
    y = ops.grouped_linear(xd, wd, plan, zero_fill=extra_rows > 0)
    assert y.shape == (Rn, O) and y.dtype == dtype
    y.backward(gy.to(DEV))
    # one rounding of an fp32-accumulated sum in bf16; fp32 sums within 1e-5 of the largest value
    tol, metric = (1e-5, rel_max) if dtype == torch.float32 else (5e-3, rel_l2)
    for name, got, want in (("y", y[:covered], want_y), ("dx", xd.grad[:covered], want_dx), ("dw", wd.grad, want_dw)):
        assert got.shape == want.shape, name
        if want.numel() == 0 or want.abs().max() == 0:
            assert got.numel() == 0 or got.abs().max() == 0, name
        else:
            assert metric(got, want) < tol, f"{name} {metric(got, want)}"
    if extra_rows:
        assert not y[covered:].any() and not xd.grad[covered:].any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("counts,I,O", [((5, 6, 4, 7), 16, 32), ((2, 0, 3), 4, 8), ((0, 5, 0), 8, 4), ((0, 0, 0), 4, 8),
                                        ((130, 1, 64, 300), 72, 40), ((100, 0, 29), 40, 72)])
def test_grouped_linear_generic(ops, dtype, counts, I, O):
    print(f"grouped linear generic {dtype} {counts} I={I} O={O}", flush=True)
    _linear_case(ops, dtype, counts, I, O)


@pytest.mark.parametrize("counts,I,O", [
    ((200, 0, 129), 384, 768), ((131, 260), 768, 384), ((1000,), 384, 512), ((3,), 384, 384),
    ((513, 77, 0, 256, 255, 257, 1), 512, 448), ((0, 0, 0), 384, 384),
    # few row tiles: the input gradient runs on 128-column tiles
    ((4096,), 448, 2048), ((700, 900), 2048, 384),
    ((300, 0, 5, 700, 1, 64, 65, 0, 128, 129, 2, 5, 4, 250, 0, 90, 17, 33, 640), 640, 384),
])
def test_grouped_linear_bf16_mfma(ops, counts, I, O):
    print(f"grouped linear bf16 mfma {counts} I={I} O={O}", flush=True)
    _linear_case(ops, torch.bfloat16, counts, I, O)


@pytest.mark.parametrize("dtype,I,O", [(torch.float32, 16, 24), (torch.bfloat16, 384, 448)])
def test_grouped_linear_zero_fills_rows_the_counts_do_not_cover(ops, dtype, I, O):
    print(f"grouped linear uncovered rows {dtype}", flush=True)
    _linear_case(ops, dtype, (10, 0, 20), I, O, extra_rows=10)


def test_grouped_linear_needs_only_the_gradients_asked_for(ops):
    print("grouped linear partial gradients", flush=True)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(50, 384, generator=g).bfloat16().to(DEV)
    w = (torch.randn(2, 448, 384, generator=g) * 0.1).bfloat16().to(DEV)
    plan = ops.segments_from_counts(torch.tensor([20, 30], dtype=torch.int32, device=DEV), 50)
    gy = torch.randn(50, 448, generator=g).bfloat16().to(DEV)
    full = ops.grouped_linear_bwd(gy, x, w, plan)
    only_dx = ops.grouped_linear_bwd(gy, x, w, plan, need_dw=False)
    only_dw = ops.grouped_linear_bwd(gy, x, w, plan, need_dx=False)
    assert torch.equal(only_dx[0], full[0]) and only_dx[1] is None
    assert torch.equal(only_dw[1], full[1]) and only_dw[0] is None
    assert ops.grouped_linear(x, w, plan).requires_grad is False


@pytest.mark.parametrize("dtype,counts,D,Fd", [(torch.float32, (5, 6, 4, 7), 16, 32), (torch.bfloat16, (200, 0, 129), 384, 768),
                                               (torch.bfloat16, (100, 0, 29), 72, 40)])
def test_grouped_experts_module_with_the_situ_activation(ops, dtype, counts, D, Fd):
    """GroupedExperts(activation_fn=SituGLU(...)) called with counts, as the reference's
    dispatchers call it (experts.py:152-209), against the oracle with the restated formula."""
    from torchllmtuner_amd import moe

    print(f"experts situ {dtype} {counts} D={D} F={Fd}", flush=True)
    g = torch.Generator().manual_seed(9)
    El, Rn = len(counts), sum(counts)
    x = torch.randn(Rn, D, generator=g).to(dtype)
    ws = [(torch.randn(El, Fd, D, generator=g) * 0.1).to(dtype), (torch.randn(El, Fd, D, generator=g) * 0.1).to(dtype),
          (torch.randn(El, D, Fd, generator=g) * 0.1).to(dtype)]
    gy = torch.randn(Rn, D, generator=g).to(dtype)
    ref_in = [t.clone().requires_grad_() for t in (x, *ws)]
    ref = R.grouped_experts(ref_in[0], torch.tensor(counts), *ref_in[1:], lambda a, b: R.situ_glu(a, b, 1.5, None))
    ref.backward(gy)
    experts = moe.GroupedExperts(D, Fd, El, activation_fn=moe.SituGLU(1.5)).to(DEV).to(dtype)
    with torch.no_grad():
        for prm, t in zip((experts.w1_EFD, experts.w3_EFD, experts.w2_EDF), ws):
            prm.copy_(t)
    xd = x.to(DEV).requires_grad_()
    y = experts(xd, torch.tensor(counts, device=DEV))
    y.backward(gy.to(DEV))
    tol, metric = (FP32_TOL, rel_max) if dtype == torch.float32 else (BF16_TOL, rel_l2)
    for name, got, want in (("y", y, ref), ("dx", xd.grad, ref_in[0].grad), ("dw1", experts.w1_EFD.grad, ref_in[1].grad),
                            ("dw3", experts.w3_EFD.grad, ref_in[2].grad), ("dw2", experts.w2_EDF.grad, ref_in[3].grad)):
        if want.abs().max() == 0:
            assert got.abs().max() == 0, name
        else:
            assert metric(got, want) < tol, f"{name} {metric(got, want)}"


def test_a_subclass_with_its_own_grouped_mm_gets_the_reference_arguments(ops):
    """``GroupedExperts._grouped_mm(x, weight_EOI, offsets_E)`` is the reference's pluggable product
    (experts.py:211-216): an override is called for all three projections -- SwiGLU included, which
    then runs as the activation module between them -- with the cumulative int32 end offsets the
    reference passes, and the result equals the built-in kernels'."""
    from torchllmtuner_amd import moe

    print("experts with an overridden _grouped_mm", flush=True)
    seen = []

    class LoopExperts(moe.GroupedExperts):
        def _grouped_mm(self, x_TD, weight_EOI, offsets_E):
            seen.append((tuple(x_TD.shape), tuple(weight_EOI.shape), offsets_E.dtype, offsets_E.cpu().tolist()))
            out = x_TD.new_zeros(x_TD.shape[0], weight_EOI.shape[1])
            start = 0
            for e, end in enumerate(offsets_E.cpu().tolist()):  # the loop path of experts.py:272-285
                out[start:end] = F.linear(x_TD[start:end], weight_EOI[e])
                start = end
            return out

    torch.manual_seed(4)
    counts, D, Fd = (37, 0, 90, 1), 384, 448
    mine = LoopExperts(D, Fd, len(counts)).to(DEV).to(torch.bfloat16)
    builtin = moe.GroupedExperts(D, Fd, len(counts)).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        for p in mine.parameters():
            p.normal_(0, 0.05)
        builtin.load_state_dict(mine.state_dict())
    assert builtin.fuses_activation() and not mine.fuses_activation()
    x = torch.randn(sum(counts), D, device=DEV).bfloat16()
    cnt = torch.tensor(counts, device=DEV)
    xa, xb = x.clone().requires_grad_(), x.clone().requires_grad_()
    ya, yb = mine(xa, cnt), builtin(xb, cnt)
    assert [s[:3] for s in seen] == [((128, D), (4, Fd, D), torch.int32)] * 2 + [((128, Fd), (4, D, Fd), torch.int32)]
    assert all(s[3] == [37, 37, 127, 128] for s in seen)
    assert rel_l2(ya, yb) < BF16_TOL
    gy = torch.randn_like(ya)
    ya.backward(gy)
    yb.backward(gy)
    assert rel_l2(xa.grad, xb.grad) < BF16_TOL
    for pa, pb in zip(mine.parameters(), builtin.parameters()):
        assert rel_l2(pa.grad, pb.grad) < BF16_TOL


@pytest.mark.parametrize("dtype,D,Fd,align", [(torch.float32, 96, 160, 1), (torch.bfloat16, 72, 40, 8), (torch.float64, 24, 40, 1),
                                              (torch.bfloat16, 384, 448, 1)])
def test_rows_experts_combine_is_the_three_stages_in_one_operator(ops, dtype, D, Fd, align):
    """The one-operator form of scatter -> experts -> combine (what the module layer runs where the
    folded kernels do not apply) gives the output and every gradient of the three differentiable
    stages composed by hand, bit for bit."""
    print(f"rows_experts_combine {dtype} D={D} F={Fd} align={align}", flush=True)
    T, K, E = 300, 4, 8
    g = torch.Generator().manual_seed(13)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(DEV)
    mk = lambda *s: (torch.randn(*s, generator=g, dtype=torch.float64) * 0.1).to(dtype).to(DEV)
    leaves_a = [torch.randn(T, D, generator=g, dtype=torch.float64).to(dtype).to(DEV), torch.rand(T, K, generator=g).to(DEV),
                mk(E, Fd, D), mk(E, Fd, D), mk(E, D, Fd)]
    leaves_b = [t.clone() for t in leaves_a]
    for t in leaves_a + leaves_b:
        t.requires_grad_()
    dout = torch.randn(T, D, generator=g, dtype=torch.float64).to(dtype).to(DEV)
    plan = ops.permute_plan(ids, E, 0, E, align)
    one = ops.rows_experts_combine(*leaves_a, plan)
    x, wts, w1, w3, w2 = leaves_b
    three = ops.combine(ops.grouped_swiglu(ops.permute_rows(x, plan), w1, w3, w2, plan), wts, plan)
    assert torch.equal(one, three)
    one.backward(dout)
    three.backward(dout)
    for a, b in zip(leaves_a, leaves_b):
        assert torch.equal(a.grad, b.grad)
    # only the scores ask for a gradient
    w_only = leaves_a[1].detach().clone().requires_grad_()
    ops.rows_experts_combine(leaves_a[0].detach(), w_only, *(t.detach() for t in leaves_a[2:]), plan).backward(dout)
    assert torch.equal(w_only.grad, leaves_b[1].grad)


# ---------------------------------------------------------------- balance loss
@pytest.mark.parametrize("seed", [0, 1])
def test_grouped_experts_bf16_mfma_random_segments(ops, seed):
    """Twenty seeded random segment lists per seed on the MFMA path: widths with odd and even
    numbers of 64-wide K steps, one to seventeen experts, counts around every tile and block
    boundary (0, 1, 15..17, 63..65, 255..257, 511..513, 1100)."""
    import random

    rng = random.Random(seed)
    sizes = [0, 0, 1, 3, 15, 16, 17, 63, 64, 65, 200, 255, 256, 257, 300, 511, 512, 513, 700, 1100]
    for it in range(20):
        D, Fd = rng.choice([384, 448, 512, 640, 1024]), rng.choice([384, 448, 576, 768])
        counts = tuple(rng.choice(sizes) for _ in range(rng.choice([1, 2, 3, 5, 9, 17])))
        if sum(counts) > 4000:
            counts = tuple(c // 3 for c in counts)
        print(f"experts bf16 mfma random {seed}/{it}: D={D} F={Fd} counts={counts}", flush=True)
        _experts_case(ops, torch.bfloat16, counts, D, Fd, std=0.05, seed=100 * seed + it)


@pytest.mark.parametrize("T,E,K,padded", [(12, 4, 2, False), (1000, 128, 8, True), (4096, 256, 8, True),
                                          (0, 8, 2, False), (77, 320, 5, False)])
def test_balance_loss_fwd_bwd(ops, T, E, K, padded):
    print(f"balance loss T={T} E={E}", flush=True)
    g = torch.Generator().manual_seed(3)
    s = torch.rand(T, E, generator=g)
    m = torch.zeros(T, E, dtype=torch.bool)
    if T:
        m.scatter_(-1, torch.topk(s, K).indices, True)
    pad = None
    if padded:
        pad = torch.rand(T, generator=g) < 0.1
        m &= ~pad[:, None]
    sr = s.clone().requires_grad_()
    ref = R.balance_loss(sr, m, pad)
    loss, f_E = ops.balance_loss_fwd(s.to(DEV), m.to(DEV), None if pad is None else pad.to(DEV))
    assert abs(float(loss) - float(ref.detach())) <= 1e-5 * max(1.0, abs(float(ref.detach())))
    if T == 0:
        return
    ref.backward()
    grad = ops.balance_loss_bwd(s.to(DEV), f_E, torch.tensor(1.0, device=DEV), None if pad is None else pad.to(DEV))
    assert rel_max(grad, sr.grad) < FP32_TOL
    # twice the upstream gradient, twice the result
    grad2 = ops.balance_loss_bwd(s.to(DEV), f_E, torch.tensor(2.0, device=DEV), None if pad is None else pad.to(DEV))
    assert torch.equal(grad2, grad * 2)


# ------------------------------------------- experts + combine, one backward for both
@pytest.mark.parametrize("T,K,E,D,Fd,align,local,skew", [
    (700, 4, 16, 384, 768, 1, None, False),     # F a multiple of the 256-column dH tile
    (700, 4, 16, 512, 448, 8, None, False),     # last dH tile starts early: shared columns counted once
    (1500, 8, 32, 384, 384, 1, (8, 24), True),  # local expert range, skewed counts, dropped slots
    (64, 2, 8, 384, 640, 128, None, False),     # few rows per expert, padded segments
])
def test_folded_combine_backward_matches_the_two_call_backward(ops, T, K, E, D, Fd, align, local, skew):
    """mi355_grouped_swiglu_combine_bwd against mi355_combine_bwd + mi355_grouped_swiglu_bwd on
    the same inputs (both bf16, two rounding points apart), and both against the fp32 oracle."""
    print(f"folded combine bwd T={T} K={K} E={E} D={D} F={Fd} align={align} local={local} skew={skew}", flush=True)
    g = torch.Generator().manual_seed(11)
    if skew:
        pr = torch.arange(1, E + 1, dtype=torch.float32) ** -1.2
        ids = torch.stack([torch.multinomial(pr, K, generator=g) for _ in range(T)])
    else:
        ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)])
    weights = torch.rand(T, K, generator=g) + 0.05
    weights = weights / weights.sum(-1, keepdim=True)
    lo, hi = local if local else (0, E)
    El = hi - lo
    x = torch.randn(T, D, generator=g).bfloat16()
    dout = torch.randn(T, D, generator=g).bfloat16()
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).bfloat16()
    w1, w3, w2 = mk(El, Fd, D), mk(El, Fd, D), mk(El, D, Fd)

    plan = ops.permute_plan(ids.to(DEV), E, align=align, local_lo=lo, local_hi=hi)
    assert ops.combine_bwd_slots(torch.bfloat16, D, Fd) > 0
    xd, wd, dd = x.to(DEV), weights.to(DEV), dout.to(DEV)
    w1d, w3d, w2d = w1.to(DEV), w3.to(DEV), w2.to(DEV)
    y, gate, up, h = ops.grouped_swiglu_fwd(xd, w1d, w3d, w2d, plan, gather=True)

    dy, dwt_a = ops.combine_bwd(dd, y, wd, plan)
    drows_a, dw1_a, dw3_a, dw2_a = ops.grouped_swiglu_bwd(dy, xd, w1d, w3d, w2d, gate, up, h, plan, gather=True)
    scale = ops.combine_row_scale(wd, plan)
    dx_b, dw1_b, dw3_b, dw2_b, dwt_b = ops.grouped_swiglu_combine_bwd(dd, xd, wd, w1d, w3d, w2d, gate, up, plan)

    # row_scale is the weights read through the plan, zero where a row holds padding
    sor = plan.slot_of_row.cpu()
    want_scale = torch.where(sor >= 0, weights.flatten()[sor.clamp(min=0)], torch.zeros(()))
    assert torch.equal(scale.cpu(), want_scale)

    dx_a = ops.permute_rows_bwd(drows_a, plan)
    for name, a, b in (("dx", dx_a, dx_b), ("dw1", dw1_a, dw1_b), ("dw3", dw3_a, dw3_b), ("dw2", dw2_a, dw2_b),
                       ("dweights", dwt_a, dwt_b)):
        assert rel_l2(b, a) < BF16_TOL, f"{name}: folded vs two calls {rel_l2(b, a)}"

    # the fp32 oracle of the whole thing: out = sum_k w * experts(x)[row], gradients by autograd
    xr, wr = x.float().requires_grad_(), weights.clone().requires_grad_()
    p1, p3, p2 = (w.float().requires_grad_() for w in (w1, w3, w2))
    out = torch.zeros(T, D)
    flat = ids.flatten()
    for e in range(lo, hi):
        sel = (flat == e).nonzero().squeeze(-1)
        if sel.numel() == 0:
            continue
        tok = sel // K
        hh = F.silu(xr[tok] @ p1[e - lo].T) * (xr[tok] @ p3[e - lo].T)
        out = out.index_add(0, tok, (hh @ p2[e - lo].T) * wr.flatten()[sel, None])
    out.backward(dout.float())
    local_slot = ((ids >= lo) & (ids < hi))
    for name, got, want in (("dx", dx_b, xr.grad), ("dw1", dw1_b, p1.grad), ("dw3", dw3_b, p3.grad),
                            ("dw2", dw2_b, p2.grad), ("dweights", dwt_b, wr.grad)):
        assert rel_l2(got, want) < BF16_TOL, f"{name}: folded vs fp32 oracle {rel_l2(got, want)}"
    # slots that were dropped (experts outside the local range) get exactly zero
    assert torch.equal(dwt_b.cpu()[~local_slot], torch.zeros_like(dwt_b.cpu()[~local_slot]))


def test_gathered_experts_combine_autograd_matches_the_explicit_backward(ops):
    """The differentiable operator (forward + registered autograd formula) gives the gradients of
    the explicit backward call, bit for bit, and leaves unrequested gradients alone."""
    print("gather_experts_combine autograd", flush=True)
    T, K, E, D, Fd = 300, 4, 8, 384, 384
    g = torch.Generator().manual_seed(3)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(DEV)
    wts = torch.rand(T, K, generator=g).to(DEV).requires_grad_()
    x = torch.randn(T, D, generator=g).bfloat16().to(DEV).requires_grad_()
    dout = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).bfloat16().to(DEV).requires_grad_()
    w1, w3, w2 = mk(E, Fd, D), mk(E, Fd, D), mk(E, D, Fd)
    plan = ops.permute_plan(ids, E)
    out = ops.gather_experts_combine(x, wts, w1, w3, w2, plan)
    out.backward(dout)
    with torch.no_grad():
        y, gate, up, h = ops.grouped_swiglu_fwd(x, w1, w3, w2, plan, gather=True)
        assert torch.equal(out, ops.combine_fwd(y, wts, plan))
        dx, dw1, dw3, dw2, dwt = ops.grouped_swiglu_combine_bwd(dout, x, wts, w1, w3, w2, gate, up, plan)
    for got, want in ((x.grad, dx), (w1.grad, dw1), (w3.grad, dw3), (w2.grad, dw2), (wts.grad, dwt)):
        assert torch.equal(got, want)
    # only dx asked for: the weight-gradient kernels do not run and nothing else gets a gradient
    x2 = x.detach().clone().requires_grad_()
    ops.gather_experts_combine(x2, wts.detach(), w1.detach(), w3.detach(), w2.detach(), plan).backward(dout)
    assert torch.equal(x2.grad, dx)


def test_fused_backward_forks_and_joins_on_the_callers_stream(ops):
    """The fused backward runs its weight gradients on a second stream and joins before it
    returns: on a caller's own stream, several times in a row, with the gradients consumed by the
    very next launch, every gradient equals the first run's bit for bit (a missing join would let
    the consumer read weight gradients that are still being written)."""
    print("gather_experts_combine on a caller's stream", flush=True)
    T, K, E, D, Fd = 2048, 4, 8, 512, 768
    g = torch.Generator().manual_seed(11)
    ids = torch.stack([torch.randperm(E, generator=g)[:K] for _ in range(T)]).to(DEV)
    wts = torch.rand(T, K, generator=g).to(DEV)
    x = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    dout = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    mk = lambda *s: (torch.randn(*s, generator=g) * 0.05).bfloat16().to(DEV)
    w1, w3, w2 = mk(E, Fd, D), mk(E, Fd, D), mk(E, D, Fd)
    plan = ops.permute_plan(ids, E)

    def grads():
        leaves = [t.detach().clone().requires_grad_() for t in (x, wts, w1, w3, w2)]
        ops.gather_experts_combine(*leaves, plan).backward(dout)
        # consumed at once, on the same stream
        return [t.grad.clone() for t in leaves], torch.stack([t.grad.float().sum() for t in leaves])

    first, first_sums = grads()
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for it in range(5):
            again, sums = grads()
            for a, b in zip(again, first):
                assert torch.equal(a, b), f"iteration {it}"
            assert torch.equal(sums, first_sums), f"iteration {it}"
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()


@pytest.mark.parametrize("counts", [(2, 0, 3), (0, 5, 0), (0, 0, 0)])
@pytest.mark.parametrize("dtype,D,Fd", [(torch.float32, 4, 8), (torch.float64, 4, 8), (torch.bfloat16, 384, 384)])
def test_grouped_experts_under_torch_compile(counts, dtype, D, Fd):
    """GroupedExperts traced whole (aot_eager, fullgraph) equals eager, forward and gradients, for
    the zero-count segment cases of tests/unit_tests/cpu/test_expert_compile_segments.py:13-40:
    the operators carry fake kernels and registered autograd formulas, so nothing graph-breaks."""
    print(f"experts under torch.compile {counts} {dtype}", flush=True)
    from torchllmtuner_amd import moe

    torch.manual_seed(0)
    El, Rn = len(counts), sum(counts)
    experts = moe.GroupedExperts(D, Fd, El).to(DEV).to(dtype)
    with torch.no_grad():
        for p in experts.parameters():
            p.normal_(0, 0.1)
    x = torch.randn(Rn, D, device=DEV).to(dtype)
    cnt = torch.tensor(counts, device=DEV)
    gy = torch.randn(Rn, D, device=DEV).to(dtype)

    def run(fn):
        experts.zero_grad(set_to_none=True)
        xin = x.clone().requires_grad_()
        y = fn(xin, cnt)
        y.backward(gy)
        return [y.detach(), xin.grad] + [p.grad.clone() for p in experts.parameters()]

    eager = run(experts)
    torch._dynamo.reset()
    compiled = run(torch.compile(experts, backend="aot_eager", fullgraph=True))
    for a, b in zip(eager, compiled):
        assert a.shape == b.shape and torch.equal(a, b)


def test_rows_not_covered_by_the_counts_come_back_as_zeros(ops):
    """Counts that add up to fewer rows than were passed (the reference asserts; here the device
    clamps): the uncovered rows of the output and of the input gradient are zeros, never
    uninitialised memory."""
    from torchllmtuner_amd import moe

    torch.manual_seed(1)
    experts = moe.GroupedExperts(384, 384, 3).to(DEV).to(torch.bfloat16)
    with torch.no_grad():
        for p in experts.parameters():
            p.normal_(0, 0.1)
    x = torch.randn(40, 384, device=DEV).bfloat16().requires_grad_()
    # poison the allocator's free blocks so that "uninitialised" cannot happen to be zero
    junk = torch.full((40, 384), float("nan"), device=DEV, dtype=torch.bfloat16)
    del junk
    y = experts(x, torch.tensor([10, 0, 20], device=DEV))
    assert torch.isfinite(y.float()).all() and not y[30:].any() and y[:30].any()
    y.backward(torch.ones_like(y))
    assert torch.isfinite(x.grad.float()).all() and not x.grad[30:].any()


def test_plan_edge_cases_largest_expert_count_and_ids_out_of_range(ops):
    """E = 2048, the largest expert count the plan accepts (its scan keeps 56 KiB in LDS there),
    is still the stable argsort; one more expert is refused; a slot whose id lies outside [0, E)
    is not counted and gets no row."""
    g = torch.Generator().manual_seed(2)
    T, K, E = 1500, 4, 2048
    ids = torch.randint(0, E, (T, K), generator=g)
    plan = ops.permute_plan(ids.to(DEV), E)
    assert torch.equal(plan.counts_E.cpu().long(), torch.bincount(ids.reshape(-1), minlength=E))
    assert torch.equal(plan.slot_of_row.cpu().long(), torch.argsort(ids.reshape(-1), stable=True))
    with pytest.raises(ValueError, match="exceeds 2048"):
        ops.permute_plan(ids.to(DEV), E + 1)
    E = 8
    ids = torch.randint(0, E, (64, 2), generator=g)
    bad = ids.clone()
    bad[3, 1], bad[17, 0] = E, -1
    plan = ops.permute_plan(bad.to(DEV), E)
    keep = (bad >= 0) & (bad < E)
    assert torch.equal(plan.counts_E.cpu().long(), torch.bincount(bad[keep], minlength=E))
    ros = plan.row_of_slot.cpu().view(64, 2)
    assert ros[3, 1] == -1 and ros[17, 0] == -1 and int((ros >= 0).sum()) == 126
    assert int(plan.total_rows) == 126
