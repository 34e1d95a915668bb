"""The committed known-answer vectors (tests/golden/known_answers.json), each a literal
from one of the reference's own tests, checked twice: the CPU oracle (not gpu) and the HIP
kernels through the C ABI (gpu).  Integer results must match exactly; the float vectors
are exact in fp32 up to the last few ulps, checked at 1e-6 relative."""

import json
import os

import pytest
import torch

from oracle import moe_ref as R

DEV = "cuda:0"
with open(os.path.join(os.path.dirname(__file__), "golden", "known_answers.json")) as fh:
    G = json.load(fh)


def _close(got, want):
    torch.testing.assert_close(got.detach().cpu().float(), torch.tensor(want, dtype=torch.float32),
                               rtol=1e-6, atol=1e-6)


def _logit(scores):
    s = torch.tensor(scores)
    return torch.log(s.clamp_min(1e-6) / (1 - s).clamp_min(1e-6))  # sigmoid^-1, order-preserving


# ------------------------------------------------------------------ oracle
@pytest.mark.parametrize("case", G["stable_permute"], ids=lambda c: c["source"][:48])
def test_oracle_stable_permute(case):
    x = torch.tensor(case["x"], dtype=torch.float64, requires_grad=True)
    ids = torch.tensor(case["expert_ids"])
    rows, tok, _, _ = R.local_reorder(x, torch.ones(ids.shape, dtype=torch.float64), ids)
    assert tok.tolist() == case["source_rows"]
    assert torch.equal(rows, x[case["source_rows"]])
    if case["row_grad"] is not None:
        (rows * torch.tensor(case["row_grad"], dtype=torch.float64)).sum().backward()
        assert torch.equal(x.grad, torch.tensor(case["x_grad"], dtype=torch.float64))


@pytest.mark.parametrize("case", G["group_limited_select"])
def test_oracle_group_limited_select(case):
    ids = R.select_experts(torch.tensor(case["scores"]), None, case["top_k"],
                           case["num_expert_groups"], case["num_limited_groups"])
    assert ids.tolist() == case["expert_ids"]


@pytest.mark.parametrize("case", G["fixed_routing"], ids=lambda c: c["mode"])
def test_oracle_fixed_routing(case):
    spec = R.RouterSpec(case["num_experts"], case["top_k"], route_scale=3.0,
                        fixed_router=case["mode"] == "fixed",
                        debug_force_load_balance=case["mode"] == "balanced")
    w, ids, _ = R.route(torch.randn(case["num_tokens"], case["num_experts"]), spec)
    assert ids.tolist() == case["expert_ids"]
    if case["weights"] is not None:
        assert torch.equal(w, torch.tensor(case["weights"]))


@pytest.mark.parametrize("case", G["router_gate"])
def test_oracle_router_gate(case):
    w = torch.tensor(case["weight"], dtype=torch.float64, requires_grad=True)
    x = torch.tensor(case["x"], dtype=torch.float64, requires_grad=True)
    out = R.router_gate(x, w)
    assert out.dtype == torch.float32
    _close(out, case["logits_fp32"])
    out.sum().backward()
    assert x.grad.dtype == torch.float64 and w.grad.dtype == torch.float64
    _close(x.grad, case["x_grad_for_ones"])
    _close(w.grad, case["weight_grad_for_ones"])


@pytest.mark.parametrize("case", G["weighted_combine"], ids=lambda c: c["source"][:48])
def test_oracle_weighted_combine(case):
    tokens = torch.tensor(case["tokens"], requires_grad=True)
    ids = torch.tensor(case["expert_ids"])
    scores = torch.tensor(case["scores"], requires_grad=True)
    rows, tok, s_sorted, perm = R.local_reorder(tokens, scores, ids)
    gains = (ids.reshape(-1)[perm] + 1).unsqueeze(1)
    out = R.combine(rows * gains, tok, s_sorted, tokens)
    _close(out, case["out"])
    (g_scores,) = torch.autograd.grad(out.sum(), scores)
    _close(g_scores, case["score_grad_for_ones"])


@pytest.mark.parametrize("case", G["padded_permute"])
def test_oracle_padded_permute(case):
    ids = torch.tensor(case["expert_ids"])
    T, K = ids.shape
    x = torch.arange(1, T + 1, dtype=torch.float32)[:, None].expand(T, 2).contiguous()
    rows, tok, _, _ = R.local_reorder(x, torch.ones(T, K), ids)
    counts = torch.bincount(ids.reshape(-1), minlength=case["num_experts"])
    _, padded, pidx, pc = R.permute_and_pad(rows, counts, case["pad_multiple"])
    assert pc.tolist() == case["padded_counts"]
    tok_ext = torch.cat([tok, torch.tensor([-1])])
    assert tok_ext[pidx].tolist() == case["token_of_row"]
    want = torch.tensor([0.0 if t < 0 else t + 1.0 for t in case["token_of_row"]])
    assert torch.equal(padded[:, 0], want)


# ------------------------------------------------------------------ HIP path
@pytest.fixture(scope="module")
def ops():
    from torchllmtuner_amd import ops as _ops

    return _ops


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["stable_permute"], ids=lambda c: c["source"][:48])
def test_gpu_stable_permute(ops, case):
    x = torch.tensor(case["x"], dtype=torch.float32, device=DEV)
    ids = torch.tensor(case["expert_ids"], device=DEV)
    plan = ops.permute_plan(ids, int(ids.max()) + 1)
    assert plan.token_of_row.cpu().tolist() == case["source_rows"]
    rows = ops.permute_rows_fwd(x, plan)
    assert torch.equal(rows.cpu(), x.cpu()[case["source_rows"]])
    if case["row_grad"] is not None:
        dx = ops.permute_rows_bwd(torch.tensor(case["row_grad"], dtype=torch.float32, device=DEV), plan)
        assert torch.equal(dx.cpu(), torch.tensor(case["x_grad"], dtype=torch.float32))


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["group_limited_select"])
def test_gpu_group_limited_select(ops, case):
    _, ids, _ = ops.router_select_fwd(_logit(case["scores"]).to(DEV), None, case["top_k"], "sigmoid",
                                      False, 1.0, case["num_expert_groups"], case["num_limited_groups"])
    assert ids.cpu().tolist() == case["expert_ids"]


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["fixed_routing"], ids=lambda c: c["mode"])
def test_gpu_fixed_routing(ops, case):
    mode = ops.SELECT_FIXED if case["mode"] == "fixed" else ops.SELECT_BALANCED
    logits = torch.randn(case["num_tokens"], case["num_experts"], device=DEV)
    w, ids, _ = ops.router_select_fwd(logits, None, case["top_k"], "sigmoid", False, 3.0, mode=mode)
    assert ids.cpu().tolist() == case["expert_ids"]
    if case["weights"] is not None:
        assert torch.equal(w.cpu(), torch.tensor(case["weights"]))
    else:
        assert torch.equal(w.cpu(), (torch.sigmoid(logits).gather(-1, ids) * 3.0).cpu())


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["router_gate"])
def test_gpu_router_gate(ops, case):
    w = torch.tensor(case["weight"], dtype=torch.float32, device=DEV)
    x = torch.tensor(case["x"], dtype=torch.float64).float().to(DEV)
    out = ops.router_gate_fwd(x, w)
    assert out.dtype == torch.float32
    _close(out, case["logits_fp32"])
    dx, dw = ops.router_gate_bwd(torch.ones_like(out), x, w)
    _close(dx, case["x_grad_for_ones"])
    _close(dw, case["weight_grad_for_ones"])


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["weighted_combine"], ids=lambda c: c["source"][:48])
def test_gpu_weighted_combine(ops, case):
    tokens = torch.tensor(case["tokens"], device=DEV)
    ids = torch.tensor(case["expert_ids"], device=DEV)
    scores = torch.tensor(case["scores"], device=DEV)
    plan = ops.permute_plan(ids, int(ids.max()) + 1)
    rows = ops.permute_rows_fwd(tokens, plan)
    gains = (ids.reshape(-1)[plan.slot_of_row.long()] + 1).unsqueeze(1).float()
    y = rows * gains
    _close(ops.combine_fwd(y, scores, plan, round_terms=False), case["out"])
    _, dscores = ops.combine_bwd(torch.ones_like(tokens), y, scores, plan)
    _close(dscores, case["score_grad_for_ones"])


@pytest.mark.gpu
@pytest.mark.parametrize("case", G["padded_permute"])
def test_gpu_padded_permute(ops, case):
    ids = torch.tensor(case["expert_ids"], device=DEV)
    T = ids.shape[0]
    plan = ops.permute_plan(ids, case["num_experts"], align=case["pad_multiple"])
    total = int(plan.total_rows.item())
    assert (plan.seg_offsets[1:] - plan.seg_offsets[:-1]).cpu().tolist() == case["padded_counts"]
    assert plan.token_of_row.cpu()[:total].tolist() == case["token_of_row"]
    x = torch.arange(1, T + 1, dtype=torch.float32, device=DEV)[:, None].expand(T, 4).contiguous()
    rows = ops.permute_rows_fwd(x, plan)[:total]
    want = torch.tensor([0.0 if t < 0 else t + 1.0 for t in case["token_of_row"]])
    assert torch.equal(rows[:, 0].cpu(), want)  # padding rows are zero
