"""Pin the CPU oracle against the reference's own known answers and closed forms.

Literals are the ones the reference's tests hold (file:line cited per test); the
rest are textbook identities, brute force in fp64 and invariants chosen so that a
dropped term, wrong sign/index or transposed operand fails at least one of them.
"""

import itertools

import pytest
import torch
import torch.nn.functional as F

from oracle import moe_ref as R


# ---- router gate ----------------------------------------------------------
def test_gate_equals_plain_fp32_linear_bitwise():
    # tests/unit_tests/cpu/models/test_models_common.py:53-62
    torch.manual_seed(0)
    w = torch.randn(4, 8)
    x = torch.randn(3, 8)
    assert torch.equal(R.router_gate(x, w), F.linear(x.float(), w))


def test_gate_fp32_out_from_bf16_and_bf16_grad():
    # test_models_common.py:21-51
    torch.manual_seed(0)
    w = torch.randn(4, 8).bfloat16().requires_grad_()
    x = torch.randn(3, 8).bfloat16().requires_grad_()
    out = R.router_gate(x, w)
    assert out.dtype is torch.float32 and out.shape == (3, 4)
    out.sum().backward()
    assert x.grad.dtype is torch.bfloat16 and w.grad.dtype is torch.bfloat16


def test_gate_fp64_literals():
    # test_models_common.py:65-89
    w = torch.tensor([[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]], dtype=torch.float64, requires_grad=True)
    x = torch.tensor([[1.0000000001, 2.0000000001, 3.0000000001]], dtype=torch.float64, requires_grad=True)
    out = R.router_gate(x, w)
    assert out.dtype == torch.float32
    torch.testing.assert_close(out, x.float() @ w.float().T)
    out.sum().backward()
    torch.testing.assert_close(x.grad, (torch.ones(1, 2) @ w.detach().float()).double(), rtol=0, atol=0)
    torch.testing.assert_close(w.grad, (torch.ones(2, 1) @ x.detach().float()).double(), rtol=0, atol=0)


def test_gate_logit_bias_is_added_in_fp32():
    # llmtuner/models/common/linear.py:181-182
    x = torch.randn(5, 6)
    w = torch.randn(3, 6)
    b = torch.randn(3)
    assert torch.equal(R.router_gate(x, w, b), F.linear(x, w) + b)


# ---- selection ------------------------------------------------------------
def test_topk_matches_torch_topk_as_sets_without_boundary_ties():
    # routing.py:189-191; per-row set comparison as in test_moe_routing.py:199-203
    g = torch.Generator().manual_seed(3)
    s = torch.rand(257, 64, generator=g)
    ours = R.select_experts(s, None, 6)
    theirs = torch.topk(s, 6, dim=-1, sorted=False).indices
    assert torch.equal(ours.sort(-1).values, theirs.sort(-1).values)
    # order is descending score
    v = s.gather(-1, ours)
    assert bool((v[:, :-1] >= v[:, 1:]).all())


def test_ties_go_to_the_lower_expert_index():
    s = torch.tensor([[1, 1, 1, 1, 0.5, 1, 1, 1.0]])
    assert R.select_experts(s, None, 3).tolist() == [[0, 1, 2]]
    s = torch.tensor([[0.2, 0.9, 0.9, 0.1]])
    assert R.select_experts(s, None, 2).tolist() == [[1, 2]]
    assert R.select_experts(s, None, 3).tolist() == [[1, 2, 0]]


def test_group_score_is_top2_sum_known_answer():
    # test_models_common.py:144-165
    s = torch.tensor([[0.80, 0.70, 0.00, 0.00, 0.90, 0.20, 0.00, 0.00]])
    assert R.select_experts(s, None, 2, 2, 1).tolist() == [[0, 1]]


def test_group_limited_confinement_and_nonvacuity():
    # test_models_common.py:103-141
    torch.manual_seed(0)
    s = torch.sigmoid(torch.randn(64, 8))
    ids = R.select_experts(s, None, 2, 2, 1)
    grp = ids // 4
    assert bool((grp[:, :1] == grp).all())
    ids_free = R.select_experts(s, None, 2)
    grp = ids_free // 4
    assert not bool((grp[:, :1] == grp).all())


def test_group_limited_matches_bruteforce():
    g = torch.Generator().manual_seed(5)
    T, G, P, L, K = 40, 4, 4, 2, 3
    s = torch.rand(T, G * P, generator=g) - 0.3  # negatives exercise the -inf mask
    ids = R.select_experts(s, None, K, G, L)
    for t in range(T):
        row = s[t].tolist()
        gs = []
        for gi in range(G):
            seg = sorted(row[gi * P : (gi + 1) * P], reverse=True)
            gs.append(seg[0] + seg[1])
        groups = sorted(range(G), key=lambda i: (-gs[i], i))[:L]
        cand = [e for e in range(G * P) if e // P in groups]
        want = sorted(cand, key=lambda e: (-row[e], e))[:K]
        assert ids[t].tolist() == want


def test_bias_steers_choice_not_value():
    # test_models_common.py:168-195
    torch.manual_seed(0)
    logits = torch.randn(32, 8)
    spec = R.RouterSpec(8, 2, score_func="sigmoid")
    unbiased = torch.sigmoid(logits)
    w0, ids0, _ = R.route(logits, spec)
    bias = torch.zeros(8)
    bias[5] = 10.0
    w1, ids1, _ = R.route(logits, spec, bias)
    assert int((ids1 == 5).sum()) > int((ids0 == 5).sum())
    assert torch.equal(w1, unbiased.gather(1, ids1))
    assert torch.equal(w0, unbiased.gather(1, ids0))


def test_route_norm_scale_closed_form():
    # routing.py:311-315; test_debug_force_load_balance.py:104-124
    torch.manual_seed(1)
    logits = torch.randn(16, 12)
    for fn in ("softmax", "sigmoid", "sqrtsoftplus"):
        spec = R.RouterSpec(12, 4, score_func=fn, route_norm=True, route_scale=2.5)
        w, ids, m = R.route(logits, spec)
        s = {"softmax": torch.softmax(logits, -1), "sigmoid": torch.sigmoid(logits),
             "sqrtsoftplus": F.softplus(logits).sqrt()}[fn]
        g = s.gather(-1, torch.topk(s, 4).indices)
        want = g / (g.sum(-1, keepdim=True) + 1e-20) * 2.5
        torch.testing.assert_close(w, want, rtol=0, atol=0)
        torch.testing.assert_close(w.sum(-1), torch.full((16,), 2.5))
        assert m.sum().item() == 16 * 4 and bool((m.sum(-1) == 4).all())


def test_fixed_router_and_forced_balance_closed_forms():
    # test_moe_routing.py:748-753; test_debug_force_load_balance.py:36-72
    logits = torch.randn(10, 4)
    w, ids, m = R.route(logits, R.RouterSpec(4, 2, fixed_router=True, route_scale=7.0))
    assert ids.tolist() == [[(t + k) % 4 for k in range(2)] for t in range(10)]
    assert torch.equal(w, torch.full((10, 2), 0.5))
    w, ids, m = R.route(logits, R.RouterSpec(4, 2, debug_force_load_balance=True))
    assert torch.equal(ids, torch.arange(20).reshape(10, 2) % 4)
    assert m.sum(0).tolist() == [5, 5, 5, 5]
    assert torch.equal(w, torch.sigmoid(logits).gather(-1, ids))


# ---- permute ----------------------------------------------------------------
def test_stable_permutation_known_answer_and_duplicate_backward():
    # tests/unit_tests/cpu/kernel/test_kernel_contracts.py:114-127
    x = torch.arange(12, dtype=torch.float64).reshape(3, 4).requires_grad_()
    experts = torch.tensor([[2, 0], [0, 0], [2, 1]])
    rows, tok, _, _ = R.local_reorder(x, torch.ones(3, 2, dtype=torch.float64), experts)
    assert tok.tolist() == [0, 1, 1, 2, 0, 2]
    torch.testing.assert_close(rows, x[[0, 1, 1, 2, 0, 2]], atol=0, rtol=0)
    wts = torch.arange(1, 25, dtype=x.dtype).reshape(6, 4)
    (rows * wts).sum().backward()
    want = torch.stack([wts[0] + wts[4], wts[1] + wts[2], wts[3] + wts[5]])
    torch.testing.assert_close(x.grad, want, atol=0, rtol=0)


def _routing(num_tokens=6, dim=4, num_experts=4, top_k=2, seed=0):
    # tests/unit_tests/cpu/models/test_moe_token_dispatch.py:235-246
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(num_tokens, dim, generator=g)
    ids = torch.randint(0, num_experts, (num_tokens, top_k), generator=g)
    sc = torch.rand(num_tokens, top_k, generator=g)
    counts = torch.zeros(num_experts, dtype=torch.long)
    counts.scatter_add_(0, ids.reshape(-1), torch.ones(num_tokens * top_k, dtype=torch.long))
    return x, sc, ids, counts


def test_padded_permute_invariants_and_equality_with_local_path():
    # test_moe_token_dispatch.py:249-309
    x, sc, ids, counts = _routing()
    rows, tok, s_sorted, _ = R.local_reorder(x, sc, ids)
    shape, padded_rows, pidx, pc = R.permute_and_pad(rows, counts, 4)
    assert pc.tolist() == [int(c) + (-int(c) % 4) for c in counts.tolist()]
    assert padded_rows.shape == (int(pc.sum()), x.shape[1])
    # padding rows are zero and point at the sentinel
    assert bool((padded_rows[pidx == rows.shape[0]] == 0).all())
    y = R.unpermute_padded(padded_rows * 2.0, shape, pidx)
    out_pad = R.combine(y, tok, s_sorted, x)
    out_loc = R.combine(rows * 2.0, tok, s_sorted, x)
    torch.testing.assert_close(out_pad, out_loc)
    torch.testing.assert_close(out_pad, x * (2 * sc.sum(-1, keepdim=True)))


def test_padded_permute_empty_expert_gets_no_padding():
    rows = torch.randn(5, 3)
    _, pr, pidx, pc = R.permute_and_pad(rows, torch.tensor([2, 0, 3]), 4)
    assert pc.tolist() == [4, 0, 4] and pr.shape[0] == 8
    assert pidx.tolist() == [0, 1, 5, 5, 2, 3, 4, 5]


# ---- experts ----------------------------------------------------------------
def test_grouped_experts_per_segment_hand_reference():
    # test_models_common.py:304-327
    torch.manual_seed(0)
    w1, w3 = torch.randn(4, 32, 16) * 0.03, torch.randn(4, 32, 16) * 0.03
    w2 = torch.randn(4, 16, 32) * 0.03
    x = torch.randn(22, 16)
    b = [0, 5, 11, 15, 22]
    seg = list(zip(b[:-1], b[1:]))
    want = torch.cat([(F.silu(x[s:o] @ w1[e].T) * (x[s:o] @ w3[e].T)) @ w2[e].T
                      for e, (s, o) in enumerate(seg)])
    got = R.grouped_experts(x, torch.tensor([5, 6, 4, 7]), w1, w3, w2)
    assert torch.allclose(got, want, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("counts", [(2, 0, 3), (0, 5, 0), (0, 0, 0)])
def test_zero_count_segments_fp64(counts):
    # tests/unit_tests/cpu/test_expert_compile_segments.py:13-40
    torch.manual_seed(77)
    ws = [torch.randn(3, 8, 4, dtype=torch.float64).mul_(0.1).requires_grad_() for _ in range(2)]
    w2 = torch.randn(3, 4, 8, dtype=torch.float64).mul_(0.1).requires_grad_()
    x = torch.randn(sum(counts), 4, dtype=torch.float64, requires_grad=True)
    outs = []
    for e, segx in enumerate(x.split(counts)):
        outs.append(F.linear(F.silu(F.linear(segx, ws[0][e])) * F.linear(segx, ws[1][e]), w2[e]))
    want = torch.cat(outs)
    got = R.grouped_experts(x, torch.tensor(counts), ws[0], ws[1], w2)
    torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-12)
    gw = torch.autograd.grad(want.sum(), [x, *ws, w2], allow_unused=True)
    gg = torch.autograd.grad(got.sum(), [x, *ws, w2], allow_unused=True)
    for a, b_ in zip(gg, gw):
        if b_ is None:
            assert a is None or a.count_nonzero() == 0
        else:
            torch.testing.assert_close(a, b_, rtol=1e-12, atol=1e-12)


def test_bf16_rounding_points_are_per_op():
    # experts.py:206-209: gate, up, silu, product, down each materialise in bf16
    torch.manual_seed(2)
    w1, w3 = (torch.randn(1, 8, 4) * 0.5).bfloat16(), (torch.randn(1, 8, 4) * 0.5).bfloat16()
    w2 = (torch.randn(1, 4, 8) * 0.5).bfloat16()
    x = torch.randn(6, 4).bfloat16()
    got = R.grouped_experts(x, torch.tensor([6]), w1, w3, w2)
    g = (x.float() @ w1[0].float().T).bfloat16()
    u = (x.float() @ w3[0].float().T).bfloat16()
    s = F.silu(g.float()).bfloat16()
    h = (s.float() * u.float()).bfloat16()
    want = (h.float() @ w2[0].float().T).bfloat16()
    assert got.dtype is torch.bfloat16
    torch.testing.assert_close(got.float(), want.float(), rtol=2e-2, atol=1e-3)


@pytest.mark.parametrize("linear_beta", [None, 0.0, 1.7])
def test_situ_glu_matches_the_reference_tests_explicit_formula(linear_beta):
    # tests/unit_tests/cpu/models/test_situ_activation.py:31-45: bounded gate over (1 + e^-gate),
    # times the (optionally bounded) up; values and both gradients
    torch.manual_seed(5)
    gate = torch.randn(2, 5, requires_grad=True)
    up = torch.randn(2, 5, requires_grad=True)
    got = R.situ_glu(gate, up, 2.0, linear_beta)
    bounded_gate = 2 * torch.tanh(gate / 2)
    bounded_up = up if not linear_beta else linear_beta * torch.tanh(up / linear_beta)
    want = bounded_gate / (1 + (-gate).exp()) * bounded_up
    torch.testing.assert_close(got, want)
    for a, b_ in zip(torch.autograd.grad(got.sum(), (gate, up)), torch.autograd.grad(want.sum(), (gate, up))):
        torch.testing.assert_close(a, b_)


def test_situ_glu_bounds_small_argument_limit_and_dtype():
    torch.manual_seed(6)
    g, u = torch.randn(64, 8, dtype=torch.float64) * 6, torch.randn(64, 8, dtype=torch.float64) * 6
    out = R.situ_glu(g.float(), u.float(), 1.5, 0.75)
    # |beta tanh| <= beta, sigmoid <= 1, |linear_beta tanh| <= linear_beta (equal once fp32 saturates)
    assert out.abs().max() <= 1.5 * 0.75
    # the sign is the sign of gate * up (tanh is odd, sigmoid positive)
    assert torch.equal(out.sign(), (g * u).sign().float())
    # near zero: tanh(x/b) b -> x, sigmoid -> 1/2
    eps = torch.full((4,), 1e-4, dtype=torch.float64)
    torch.testing.assert_close(R.situ_glu(eps.float(), eps.float(), 2.0, 1.0).double(), eps * eps / 2, rtol=1e-3, atol=0)
    # huge gate: beta * up exactly (both saturate), and a bf16 input comes back as bf16
    big = R.situ_glu(torch.tensor([40.0]), torch.tensor([0.5]), 3.0, None)
    assert big.item() == 1.5
    assert R.situ_glu(torch.ones(2).bfloat16(), torch.ones(2).bfloat16()).dtype is torch.bfloat16


def test_grouped_experts_with_a_callers_activation_uses_it_between_the_projections():
    # experts.py:204-209: gate, up, activation(gate, up), down -- per segment by hand
    torch.manual_seed(8)
    w1, w3 = torch.randn(3, 12, 8) * 0.3, torch.randn(3, 12, 8) * 0.3
    w2 = torch.randn(3, 8, 12) * 0.3
    x = torch.randn(9, 8)
    counts = (4, 0, 5)
    act = lambda g, u: R.situ_glu(g, u, 2.0, 1.7)
    want = torch.cat([act(sx @ w1[e].T, sx @ w3[e].T) @ w2[e].T for e, sx in enumerate(x.split(counts))])
    got = R.grouped_experts(x, torch.tensor(counts), w1, w3, w2, act)
    torch.testing.assert_close(got, want, rtol=1e-5, atol=1e-6)
    # and it is not SwiGLU
    assert not torch.allclose(got, R.grouped_experts(x, torch.tensor(counts), w1, w3, w2), atol=1e-3)


# ---- combine ----------------------------------------------------------------
def test_combine_fp64_exact():
    # test_moe_token_dispatch.py:84-99
    x = torch.tensor([[1.0000000001]], dtype=torch.float64, requires_grad=True)
    sc = torch.tensor([[0.7500000001]], dtype=torch.float64, requires_grad=True)
    rows, tok, s_sorted, _ = R.local_reorder(x, sc, torch.zeros(1, 1, dtype=torch.long))
    out = R.combine(rows, tok, s_sorted, x)
    torch.testing.assert_close(out, x * sc, rtol=0, atol=0)
    out.sum().backward()
    torch.testing.assert_close(x.grad, sc.detach(), rtol=0, atol=0)
    torch.testing.assert_close(sc.grad, x.detach(), rtol=0, atol=0)


@pytest.mark.parametrize("dtype,top_k,tokens,fp32acc", list(itertools.product(
    (torch.float32, torch.bfloat16), (2, 8), (0, 64), (False, True))))
def test_combine_matches_inverse_permute_reference(dtype, top_k, tokens, fp32acc):
    # tests/integration_tests/routed_combine_equivalence.py:22-81
    torch.manual_seed(91)
    hidden = 32
    ids = torch.randint(0, 16, (tokens, top_k))
    order = ids.flatten().argsort(stable=True)
    inverse = order.argsort()
    values = (torch.randn(tokens * top_k, hidden) * 0.1).to(dtype).requires_grad_()
    scores = torch.rand(tokens, top_k).requires_grad_()
    probe = torch.randn(tokens, hidden).to(dtype)
    tol = 2e-3 if dtype == torch.bfloat16 else 2e-6
    got = R.combine(values, order // top_k, scores.flatten()[order],
                    values.new_empty(tokens, hidden), fp32acc)
    weighted = values.float() * scores.flatten()[order, None]
    if not fp32acc:
        weighted = weighted.to(dtype)
    want = weighted[inverse].reshape(tokens, top_k, hidden).float().sum(1).to(dtype)
    torch.testing.assert_close(got, want, atol=tol, rtol=0)
    gg = torch.autograd.grad(got, (values, scores), probe, retain_graph=True)
    gw = torch.autograd.grad(want, (values, scores), probe)
    for a, b_ in zip(gg, gw):
        torch.testing.assert_close(a, b_, atol=tol, rtol=0)


def test_combine_keeps_scores_aligned_with_sorted_rows():
    # tests/unit_tests/cpu/models/test_qwen_operator_contracts.py:54-68
    tokens = torch.tensor([[1.0, 3.0], [5.0, 7.0], [11.0, 13.0]], requires_grad=True)
    experts = torch.tensor([[2, 0], [1, 2], [0, 1]])
    scores = torch.tensor([[0.1, 0.9], [0.2, 0.8], [0.7, 0.3]], requires_grad=True)
    rows, tok, s_sorted, perm = R.local_reorder(tokens, scores, experts)
    gains = (experts.reshape(-1)[perm] + 1).unsqueeze(1)
    got = R.combine(rows * gains, tok, s_sorted, tokens)
    want = tokens * (scores * (experts + 1)).sum(1, keepdim=True)
    torch.testing.assert_close(got, want)
    gg = torch.autograd.grad(got.sum(), (tokens, scores))
    gw = torch.autograd.grad(want.sum(), (tokens, scores))
    for a, b_ in zip(gg, gw):
        assert a.count_nonzero() == a.numel()
        torch.testing.assert_close(a, b_)


# ---- whole block ------------------------------------------------------------
def _params(E, D, Fd, dtype=torch.float64, seed=0, shared=False):
    g = torch.Generator().manual_seed(seed)
    mk = lambda *s: (torch.randn(*s, generator=g, dtype=torch.float64) * 0.3).to(dtype)
    p = R.MoEParams(router_w_ED=mk(E, D).float(), w1_EFD=mk(E, Fd, D), w3_EFD=mk(E, Fd, D), w2_EDF=mk(E, D, Fd))
    if shared:
        p.shared_gate_FD, p.shared_up_FD, p.shared_down_DF = mk(Fd, D), mk(Fd, D), mk(D, Fd)
    return p


def _bruteforce(x, p, spec, lo=0, hi=None):
    """Token-by-token, expert-by-expert loop in the input dtype (fp64 in tests)."""
    hi = spec.num_experts if hi is None else hi
    logits = x.float() @ p.router_w_ED.float().T
    if p.router_logit_bias_E is not None:
        logits = logits + p.router_logit_bias_E.float()
    w, ids, _ = R.route(logits, spec, p.expert_bias_E)
    out = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for k in range(spec.top_k):
            e = int(ids[t, k])
            if not lo <= e < hi:
                continue
            g = p.w1_EFD[e - lo] @ x[t]
            u = p.w3_EFD[e - lo] @ x[t]
            out[t] += (p.w2_EDF[e - lo] @ (F.silu(g) * u)) * w[t, k].to(x.dtype)
        if p.shared_gate_FD is not None:
            out[t] += p.shared_down_DF @ (F.silu(p.shared_gate_FD @ x[t]) * (p.shared_up_FD @ x[t]))
    return out


@pytest.mark.parametrize("pad", [None, 4])
@pytest.mark.parametrize("cfg", [
    dict(score_func="softmax", route_norm=True),
    dict(score_func="sigmoid", route_norm=True, route_scale=2.5, num_expert_groups=4, num_limited_groups=2),
])
def test_block_matches_bruteforce_fp64(cfg, pad):
    E, D, Fd, K, T = 8, 6, 10, 3, 17
    p = _params(E, D, Fd, shared=True)
    p.expert_bias_E = torch.linspace(-0.1, 0.1, E)
    spec = R.RouterSpec(E, K, **cfg)
    x = torch.randn(T, D, dtype=torch.float64)
    out, aux = R.moe_forward(x, p, spec, pad_multiple=pad)
    torch.testing.assert_close(out, _bruteforce(x, p, spec), rtol=1e-10, atol=1e-12)
    assert aux["counts_E"].sum().item() == T * K
    out3, _ = R.moe_forward(x.reshape(1, T, D), p, spec, pad_multiple=pad)
    assert out3.shape == (1, T, D) and torch.equal(out3.reshape(T, D), out)


def test_block_local_share_matches_bruteforce_fp64():
    E, D, Fd, K, T = 8, 6, 10, 3, 23
    full = _params(E, D, Fd)
    spec = R.RouterSpec(E, K, score_func="sigmoid", route_norm=True)
    x = torch.randn(T, D, dtype=torch.float64)
    lo, hi = 2, 5
    local = R.MoEParams(full.router_w_ED, full.w1_EFD[lo:hi], full.w3_EFD[lo:hi], full.w2_EDF[lo:hi])
    out, aux = R.moe_forward(x, local, spec, local_experts=(lo, hi))
    torch.testing.assert_close(out, _bruteforce(x, local, spec, lo, hi), rtol=1e-10, atol=1e-12)
    assert aux["counts_E"].sum().item() == T * K  # non-local assignments still counted


def test_block_analytic_experts():
    # tests/integration_tests/torchao_dispatch_equivalence.py:49-67 idea: expert e = x*(e+1)
    # realised with SwiGLU by choosing w1 so silu(gate) is a known constant is not
    # possible; instead check linearity in w2: scaling expert e's w2 by (e+1) scales
    # that expert's contribution, so out == sum_k w_k (id_k+1) y_k with unit experts.
    E, D, Fd, K, T = 4, 5, 7, 2, 11
    p = _params(E, D, Fd)
    spec = R.RouterSpec(E, K, score_func="softmax", route_norm=False)
    x = torch.randn(T, D, dtype=torch.float64)
    base, aux = R.moe_forward(x, p, spec)
    scaled = R.MoEParams(p.router_w_ED, p.w1_EFD, p.w3_EFD,
                         p.w2_EDF * torch.arange(1, E + 1, dtype=torch.float64)[:, None, None])
    out, aux2 = R.moe_forward(x, scaled, spec)
    assert torch.equal(aux["ids_TK"], aux2["ids_TK"])
    want = torch.zeros_like(x)
    for t in range(T):
        for k in range(K):
            e = int(aux["ids_TK"][t, k])
            y = p.w2_EDF[e] @ (F.silu(p.w1_EFD[e] @ x[t]) * (p.w3_EFD[e] @ x[t]))
            want[t] += aux["scores_TK"][t, k].double() * (e + 1) * y
    torch.testing.assert_close(out, want, rtol=1e-10, atol=1e-12)


# ---- per-forward load-balance loss --------------------------------------------
def _routing_from_scores(scores_TE, k):
    routing = torch.zeros_like(scores_TE, dtype=torch.bool)
    routing.scatter_(-1, torch.topk(scores_TE.detach(), k).indices, True)
    return routing


def test_balance_loss_matches_the_paper_formula_and_invariants():
    # tests/unit_tests/cpu/models/test_aux_loss.py:465-571
    torch.manual_seed(0)
    T, E, K = 12, 4, 2
    s = torch.rand(T, E)
    m = _routing_from_scores(s, K)
    counts = m.float().sum(0)
    f = (E / (K * T)) * counts                      # eq. 18 with T explicit
    p = (s / s.sum(-1, keepdim=True)).sum(0)        # eq. 19 times T
    torch.testing.assert_close(R.balance_loss(s, m), (f * p).sum(), atol=1e-6, rtol=0)
    # scale and token-order invariance
    torch.testing.assert_close(R.balance_loss(s * 1000.0, m), R.balance_loss(s, m), rtol=1e-5, atol=0)
    perm = torch.randperm(T)
    torch.testing.assert_close(R.balance_loss(s[perm], m[perm]), R.balance_loss(s, m), rtol=1e-6, atol=0)
    # even load, uniform scores: f_i = 1, sum_i p_i = T
    T2, E2 = 8, 4
    even = torch.zeros(T2, E2, dtype=torch.bool)
    even[torch.arange(T2), torch.arange(T2) % E2] = True
    assert R.balance_loss(torch.ones(T2, E2), even).item() == pytest.approx(float(T2))
    # padding rows drop out of p; the gradient reaches the scores, not the map
    pad = torch.zeros(T, dtype=torch.bool); pad[3] = pad[7] = True
    keep = ~pad
    torch.testing.assert_close(R.balance_loss(s, m & keep[:, None], pad),
                               R.balance_loss(s[keep], m[keep]), rtol=1e-6, atol=0)
    sg = s.clone().requires_grad_()
    R.balance_loss(sg, m).backward()
    assert sg.grad.abs().sum() > 0
    # closed-form gradient: (f_j - <f, s'_t>) / S_t
    S = s.sum(-1, keepdim=True)
    fE = counts / counts.sum() * E
    want = (fE[None, :] - (s / S * fE).sum(-1, keepdim=True)) / S
    torch.testing.assert_close(sg.grad, want, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- quantile-balanced routing
def test_quantile_worked_example_bins_and_estimate():
    """tests/unit_tests/cpu/models/test_moe_routing.py:233-257: E=4, K=2, 10 bins, zero bias,
    every token scored [0.92, 0.68, 0.31, 0.07] -> cutoff 0.31, required biases in bins
    1, 3, 5, 6, next bias [-0.55, -0.15, 0.25, 0.45]."""
    scores = torch.tensor([0.92, 0.68, 0.31, 0.07]).expand(4, -1)
    bias = torch.zeros(4)
    ids, cutoff = R.select_top_k_plus_one(scores, bias, 2)
    assert torch.equal(ids, torch.tensor([[0, 1]] * 4))
    assert torch.equal(cutoff, torch.full((4, 1), 0.31))
    hist = torch.zeros(4, 10, dtype=torch.int64)
    R.quantile_observe(hist, scores, cutoff, bias)
    assert hist.sum(dim=-1).tolist() == [4, 4, 4, 4]
    assert hist.nonzero().tolist() == [[0, 1], [1, 3], [2, 5], [3, 6]]
    torch.testing.assert_close(R.quantile_estimate(hist, bias, 2), torch.tensor([-0.55, -0.15, 0.25, 0.45]))


def test_quantile_histogram_counts_past_int32_and_fractional_large_counts():
    # test_moe_routing.py:357-367
    hist = torch.zeros(2, 4, dtype=torch.int64)
    hist[:, 2] = torch.iinfo(torch.int32).max
    R.quantile_observe(hist, torch.full((1, 2), 0.5), torch.full((1, 1), 0.5), torch.zeros(2))
    assert hist[:, 2].tolist() == [2147483648, 2147483648]
    # test_moe_routing.py:583-592: float32 cannot hold the half-token target, the integral
    # numerator can
    hist = torch.tensor([[8388609, 1, 0, 8388609], [8388609, 0, 1, 8388608]], dtype=torch.int64)
    got = R.quantile_estimate(hist, torch.zeros(2), 1)
    assert torch.equal(got, torch.tensor([0.125, -0.125]))


def test_quantile_empty_window_returns_the_bias_bit_for_bit():
    # test_moe_routing.py:430-441
    original = torch.tensor([-0.31, -0.12, 0.17, 0.26])
    current = original.clone()
    for _ in range(20):
        current = R.quantile_estimate(torch.zeros(4, 32, dtype=torch.int64), current, 2)
    assert torch.equal(current, original)


def test_quantile_estimate_is_mean_centred_and_pushes_toward_balance():
    # test_moe_routing.py:260-298
    g = torch.Generator().manual_seed(0)
    scores = torch.sigmoid(torch.randn(16, 4, generator=g))
    bias = torch.zeros(4)
    _, cutoff = R.select_top_k_plus_one(scores, bias, 2)
    hist = torch.zeros(4, 32, dtype=torch.int64)
    R.quantile_observe(hist, scores, cutoff, bias)
    assert abs(float(R.quantile_estimate(hist, bias, 2).sum())) < 1e-6
    # expert 0 wins every token: it must lose bias, an idle one must gain
    logits = torch.zeros(32, 4)
    logits[:, 0] = 4.0 * torch.randn(32, generator=g).abs() + 1.0
    logits[:, 1:] = 0.01 * torch.randn(32, 3, generator=g)
    scores = torch.sigmoid(logits)
    ids, cutoff = R.select_top_k_plus_one(scores, bias, 2)
    assert (ids[:, 0] == 0).all()
    hist = torch.zeros(4, 100, dtype=torch.int64)
    R.quantile_observe(hist, scores, cutoff, bias)
    nxt = R.quantile_estimate(hist, bias, 2)
    assert float(nxt[0]) < 0 and float(nxt[1:].max()) > 0


def test_quantile_observe_filters_padding_and_matches_pairwise_brute_force():
    g = torch.Generator().manual_seed(5)
    T, E, B, K = 37, 6, 17, 2
    scores = torch.sigmoid(torch.randn(T, E, generator=g))
    bias = torch.rand(E, generator=g) * 0.4 - 0.2
    pad = torch.rand(T, generator=g) < 0.3
    _, cutoff = R.select_top_k_plus_one(scores, bias, K)
    hist = torch.zeros(E, B, dtype=torch.int64)
    R.quantile_observe(hist, scores, cutoff, bias, padding_mask_T=pad)
    assert int(hist.sum()) == int((~pad).sum()) * E  # test_moe_routing.py:576
    lower = float(bias.min()) - 1.0
    width = (float(bias.max()) - float(bias.min()) + 2.0) / B
    want = torch.zeros_like(hist)
    for t in range(T):
        if pad[t]:
            continue
        for e in range(E):
            req = float(cutoff[t, 0]) - float(scores[t, e])
            want[e, min(max(int((req - lower) // width), 0), B - 1)] += 1
    # the double-precision brute force may put a pair that sits on a bin edge next door
    assert int((hist - want).abs().sum()) <= 2
    # the cutoff is the (K+1)-th largest biased score
    assert torch.equal(cutoff[:, 0], (scores + bias).sort(dim=-1, descending=True).values[:, K])


# ---------------------------------------------------------------- rms_norm (kernel registry)
def test_rms_norm_matches_the_reference_formula_gradients_and_the_library_routine():
    # tests/unit_tests/cpu/kernel/test_kernel_contracts.py:100-105
    g = torch.Generator().manual_seed(0)
    x = torch.randn(2, 3, 8, dtype=torch.float64, generator=g).requires_grad_()
    w = torch.randn(8, dtype=torch.float64, generator=g).requires_grad_()
    expected = x * torch.rsqrt(x.square().mean(-1, keepdim=True) + 1e-5) * w
    torch.testing.assert_close(R.rms_norm(x, w, 1e-5), expected)
    assert torch.autograd.gradcheck(lambda a, b: R.rms_norm(a, b, 1e-5), (x, w))
    # the reference's CPU backend is torch's own routine: equal bit for bit, rounding included
    for dtype in (torch.float32, torch.bfloat16):
        xs = (torch.randn(64, 256, generator=g) * 3).to(dtype)
        ws = torch.randn(256, generator=g).to(dtype)
        assert torch.equal(R.rms_norm(xs, ws, 1e-5), F.rms_norm(xs, (256,), ws, 1e-5))
