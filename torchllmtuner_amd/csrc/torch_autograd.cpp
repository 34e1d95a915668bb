// Autograd formulas of the differentiable `mi355_moe` operators, as C++ autograd nodes.  Each backward
// is one call of the hand-written backward operator, made through the dispatcher (so tracing and fake
// tensors see it), on the autograd engine's thread and without the interpreter lock: a small step's
// host time was mostly the interpreter's share of these nodes.
//
// In a node's backward, the returned list has one entry per forward argument, while
// needs_input_grad(i) is indexed by the i-th TENSOR among the arguments (an absent optional tensor is
// not counted).
//
// Conventions shared with ops.py: an output that was not asked for is an empty (0,) tensor; a
// gradient that is not needed is returned undefined; incoming gradients are not materialised, so
// an output nobody differentiated arrives undefined.
#include <ATen/ATen.h>
#include <ATen/core/dispatch/Dispatcher.h>
#include <torch/csrc/autograd/custom_function.h>
#include <torch/csrc/autograd/functions/utils.h>
#include <torch/library.h>

#include <optional>
#include <tuple>

namespace {

using at::Tensor;
using OptTensor = std::optional<Tensor>;
using torch::autograd::AutogradContext;
using torch::autograd::variable_list;

template <class Sig>
auto typed_op(const char* name) {
  return c10::Dispatcher::singleton().findSchemaOrThrow(name, "").typed<Sig>();
}

OptTensor opt(const Tensor& t) { return t.defined() ? OptTensor(t) : std::nullopt; }
Tensor keep(const Tensor& t, bool wanted) { return wanted ? t : Tensor(); }

// ---- router gate: dX in the input dtype, dW in the weight dtype --------------------------------
using GateFwdSig = Tensor(const Tensor&, const Tensor&, const OptTensor&);
using GateBwdSig = std::tuple<Tensor, Tensor>(const Tensor&, const Tensor&, const Tensor&, bool, bool);

struct RouterGate : public torch::autograd::Function<RouterGate> {
  static Tensor forward(AutogradContext* ctx, const Tensor& x, const Tensor& w, const OptTensor& bias) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<GateFwdSig>("mi355_moe::router_gate_fwd");
    Tensor out = op.call(x, w, bias);
    ctx->save_for_backward({x, w});
    ctx->saved_data["bias_dtype"] = bias.has_value() ? static_cast<int64_t>(bias->scalar_type()) : int64_t{-1};
    return out;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    const auto saved = ctx->get_saved_variables();
    // (needs_input_grad counts the tensors among the arguments: an absent bias has no index)
    const int64_t bias_dtype = ctx->saved_data["bias_dtype"].toInt();
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1),
               n2 = bias_dtype >= 0 && ctx->needs_input_grad(2);
    Tensor dx, dw, db;
    if (grads[0].defined()) {
      if (n0 || n1) {
        static auto op = typed_op<GateBwdSig>("mi355_moe::router_gate_bwd");
        auto r = op.call(grads[0], saved[0], saved[1], n0, n1);
        dx = keep(std::get<0>(r), n0);
        dw = keep(std::get<1>(r), n1);
      }
      if (n2 && bias_dtype >= 0) db = grads[0].to(at::kFloat).sum(0).to(static_cast<at::ScalarType>(bias_dtype));
    }
    return {dx, dw, db};
  }
};

Tensor router_gate_autograd(const Tensor& x, const Tensor& w, const OptTensor& bias) {
  if (!torch::autograd::compute_requires_grad(x, w, bias)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<GateFwdSig>("mi355_moe::router_gate_fwd");
    return op.call(x, w, bias);
  }
  return RouterGate::apply(x, w, bias);
}

// ---- selection: gather / norm / scale / score VJP per token; ids and the map carry no gradient --
using SelectFwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor>(const Tensor&, const OptTensor&, int64_t, int64_t, bool,
                                                                 double, int64_t, int64_t, int64_t, bool, bool);
using SelectBwdSig = Tensor(const Tensor&, const Tensor&, const OptTensor&, const OptTensor&, int64_t, bool, double,
                            int64_t);

struct RouterSelect : public torch::autograd::Function<RouterSelect> {
  static variable_list forward(AutogradContext* ctx, const Tensor& logits, const OptTensor& bias, int64_t K,
                               int64_t score_func, bool route_norm, double route_scale, int64_t num_groups,
                               int64_t num_limited, int64_t mode, bool want_scores, bool want_map) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<SelectFwdSig>("mi355_moe::router_select_fwd");
    auto r = op.call(logits, bias, K, score_func, route_norm, route_scale, num_groups, num_limited, mode, want_scores,
                     want_map);
    ctx->save_for_backward({logits, std::get<1>(r)});
    ctx->saved_data["score_func"] = score_func;
    ctx->saved_data["route_norm"] = route_norm;
    ctx->saved_data["route_scale"] = route_scale;
    ctx->saved_data["mode"] = mode;
    ctx->saved_data["want_scores"] = want_scores;
    ctx->set_materialize_grads(false);
    ctx->mark_non_differentiable({std::get<1>(r), std::get<3>(r)});
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(11);
    if (!ctx->needs_input_grad(0)) return out;
    const auto saved = ctx->get_saved_variables();
    static auto op = typed_op<SelectBwdSig>("mi355_moe::router_select_bwd");
    const bool want_scores = ctx->saved_data["want_scores"].toBool();
    out[0] = op.call(saved[0], saved[1], opt(grads[0]), want_scores ? opt(grads[2]) : std::nullopt,
                     ctx->saved_data["score_func"].toInt(), ctx->saved_data["route_norm"].toBool(),
                     ctx->saved_data["route_scale"].toDouble(), ctx->saved_data["mode"].toInt());
    return out;
  }
};

std::tuple<Tensor, Tensor, Tensor, Tensor> router_select_autograd(const Tensor& logits, const OptTensor& bias, int64_t K,
                                                                  int64_t score_func, bool route_norm,
                                                                  double route_scale, int64_t num_groups,
                                                                  int64_t num_limited, int64_t mode, bool want_scores,
                                                                  bool want_map) {
  if (!torch::autograd::compute_requires_grad(logits)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<SelectFwdSig>("mi355_moe::router_select_fwd");
    return op.call(logits, bias, K, score_func, route_norm, route_scale, num_groups, num_limited, mode, want_scores,
                   want_map);
  }
  auto r = RouterSelect::apply(logits, bias, K, score_func, route_norm, route_scale, num_groups, num_limited, mode,
                               want_scores, want_map);
  return {r[0], r[1], r[2], r[3]};
}

// ---- grouped experts over rows that are already in expert order ---------------------------------
using SwigluFwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor>(const Tensor&, const OptTensor&, const Tensor&,
                                                                 const Tensor&, const Tensor&, const Tensor&,
                                                                 const Tensor&, const Tensor&, const Tensor&,
                                                                 const Tensor&, int64_t, bool);
using SwigluBwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor>(const Tensor&, const Tensor&, const OptTensor&,
                                                                 const Tensor&, const Tensor&, const Tensor&,
                                                                 const Tensor&, const Tensor&, const Tensor&,
                                                                 const Tensor&, const Tensor&, const Tensor&,
                                                                 const Tensor&, const Tensor&, bool, bool, bool);

struct GroupedSwiglu : public torch::autograd::Function<GroupedSwiglu> {
  static variable_list forward(AutogradContext* ctx, const Tensor& rows, const OptTensor& tok, const Tensor& w1,
                               const Tensor& w3, const Tensor& w2, const Tensor& so, const Tensor& sc, const Tensor& te,
                               const Tensor& tr, const Tensor& nt, int64_t cap, bool zero_fill) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<SwigluFwdSig>("mi355_moe::grouped_swiglu_fwd");
    auto r = op.call(rows, tok, w1, w3, w2, so, sc, te, tr, nt, cap, zero_fill);
    ctx->save_for_backward({rows, w1, w3, w2, std::get<1>(r), std::get<2>(r), std::get<3>(r), so, sc, te, tr, nt});
    ctx->saved_data["gathered"] = tok.has_value();
    ctx->saved_data["zero_fill"] = zero_fill;
    ctx->set_materialize_grads(false);
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    TORCH_CHECK_NOT_IMPLEMENTED(
        !ctx->saved_data["gathered"].toBool(),
        "grouped_swiglu_fwd with a token gather is differentiated through gather_experts_combine_fwd");
    variable_list out(12);
    if (!grads[0].defined()) return out;
    const auto s = ctx->get_saved_variables();
    // (needs_input_grad counts the tensors among the arguments; the absent gather index is not one)
    const bool n0 = ctx->needs_input_grad(0), n2 = ctx->needs_input_grad(1), n3 = ctx->needs_input_grad(2),
               n4 = ctx->needs_input_grad(3);
    static auto op = typed_op<SwigluBwdSig>("mi355_moe::grouped_swiglu_bwd");
    auto r = op.call(grads[0], s[0], std::nullopt, s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], s[9], s[10], s[11],
                     n0, n2 || n3 || n4, ctx->saved_data["zero_fill"].toBool());
    out[0] = keep(std::get<0>(r), n0);
    out[2] = keep(std::get<1>(r), n2);
    out[3] = keep(std::get<2>(r), n3);
    out[4] = keep(std::get<3>(r), n4);
    return out;
  }
};

std::tuple<Tensor, Tensor, Tensor, Tensor> grouped_swiglu_autograd(const Tensor& rows, const OptTensor& tok,
                                                                   const Tensor& w1, const Tensor& w3, const Tensor& w2,
                                                                   const Tensor& so, const Tensor& sc, const Tensor& te,
                                                                   const Tensor& tr, const Tensor& nt, int64_t cap,
                                                                   bool zero_fill) {
  if (!torch::autograd::compute_requires_grad(rows, w1, w3, w2)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<SwigluFwdSig>("mi355_moe::grouped_swiglu_fwd");
    return op.call(rows, tok, w1, w3, w2, so, sc, te, tr, nt, cap, zero_fill);
  }
  auto r = GroupedSwiglu::apply(rows, tok, w1, w3, w2, so, sc, te, tr, nt, cap, zero_fill);
  return {r[0], r[1], r[2], r[3]};
}

// ---- row scatter + experts + combine as one node -------------------------------------------------
using RecFwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor>(
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const OptTensor&,
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, int64_t, int64_t, bool);
using RecBwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor>(
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&,
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const OptTensor&, const Tensor&, const Tensor&,
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, int64_t, int64_t, bool, bool);

struct RowsExpertsCombine : public torch::autograd::Function<RowsExpertsCombine> {
  static variable_list forward(AutogradContext* ctx, const Tensor& x, const Tensor& weights, const Tensor& w1,
                               const Tensor& w3, const Tensor& w2, const Tensor& ros, const OptTensor& sor,
                               const Tensor& total, const Tensor& so, const Tensor& sc, const Tensor& te,
                               const Tensor& tr, const Tensor& nt, int64_t K, int64_t cap, bool round_terms) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<RecFwdSig>("mi355_moe::rows_experts_combine_fwd");
    auto r = op.call(x, weights, w1, w3, w2, ros, sor, total, so, sc, te, tr, nt, K, cap, round_terms);
    // (out, rows, gate, up, h, y)
    ctx->save_for_backward({std::get<1>(r), weights, w1, w3, w2, std::get<2>(r), std::get<3>(r), std::get<4>(r),
                            std::get<5>(r), ros, sor.has_value() ? *sor : Tensor(), total, so, sc, te, tr, nt});
    ctx->saved_data["top_k"] = K;
    ctx->saved_data["num_tokens"] = x.size(0);
    ctx->set_materialize_grads(false);
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r), std::get<4>(r), std::get<5>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(16);
    if (!grads[0].defined()) return out;
    const auto s = ctx->get_saved_variables();
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1), n2 = ctx->needs_input_grad(2),
               n3 = ctx->needs_input_grad(3), n4 = ctx->needs_input_grad(4);
    static auto op = typed_op<RecBwdSig>("mi355_moe::rows_experts_combine_bwd");
    auto r = op.call(grads[0], s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], s[9], opt(s[10]), s[11], s[12],
                     s[13], s[14], s[15], s[16], ctx->saved_data["num_tokens"].toInt(),
                     ctx->saved_data["top_k"].toInt(), n0, n2 || n3 || n4);
    out[0] = keep(std::get<0>(r), n0);
    if (n1) out[1] = std::get<4>(r).to(s[1].scalar_type());
    out[2] = keep(std::get<1>(r), n2);
    out[3] = keep(std::get<2>(r), n3);
    out[4] = keep(std::get<3>(r), n4);
    return out;
  }
};

std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor> rows_experts_combine_autograd(
    const Tensor& x, const Tensor& weights, const Tensor& w1, const Tensor& w3, const Tensor& w2, const Tensor& ros,
    const OptTensor& sor, const Tensor& total, const Tensor& so, const Tensor& sc, const Tensor& te, const Tensor& tr,
    const Tensor& nt, int64_t K, int64_t cap, bool round_terms) {
  if (!torch::autograd::compute_requires_grad(x, weights, w1, w3, w2)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<RecFwdSig>("mi355_moe::rows_experts_combine_fwd");
    return op.call(x, weights, w1, w3, w2, ros, sor, total, so, sc, te, tr, nt, K, cap, round_terms);
  }
  auto r = RowsExpertsCombine::apply(x, weights, w1, w3, w2, ros, sor, total, so, sc, te, tr, nt, K, cap, round_terms);
  return {r[0], r[1], r[2], r[3], r[4], r[5]};
}

// ---- gathered experts + combine: one backward for both halves -------------------------------------
using GecFwdSig = std::tuple<Tensor, Tensor, Tensor>(const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                                                     const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                                                     const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                                                     const Tensor&, int64_t, int64_t, bool, bool);
using GecBwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor>(
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&,
    const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&,
    const Tensor&, const Tensor&, int64_t, bool, bool);

struct GatherExpertsCombine : public torch::autograd::Function<GatherExpertsCombine> {
  static variable_list forward(AutogradContext* ctx, const Tensor& x, const Tensor& weights, const Tensor& w1,
                               const Tensor& w3, const Tensor& w2, const Tensor& tok, const Tensor& sor,
                               const Tensor& ros, const Tensor& so, const Tensor& sc, const Tensor& te,
                               const Tensor& tr, const Tensor& nt, int64_t K, int64_t cap, bool round_terms,
                               bool save_gate_up) {
    TORCH_CHECK(save_gate_up,
                "gather_experts_combine_fwd was run without its gate / up outputs and cannot be differentiated");
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<GecFwdSig>("mi355_moe::gather_experts_combine_fwd");
    auto r = op.call(x, weights, w1, w3, w2, tok, sor, ros, so, sc, te, tr, nt, K, cap, round_terms, save_gate_up);
    ctx->save_for_backward({x, weights, w1, w3, w2, std::get<1>(r), std::get<2>(r), tok, sor, ros, so, sc, te, tr, nt});
    ctx->saved_data["top_k"] = K;
    ctx->set_materialize_grads(false);
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(17);
    if (!grads[0].defined()) return out;
    const auto s = ctx->get_saved_variables();
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1), n2 = ctx->needs_input_grad(2),
               n3 = ctx->needs_input_grad(3), n4 = ctx->needs_input_grad(4);
    static auto op = typed_op<GecBwdSig>("mi355_moe::gather_experts_combine_bwd");
    auto r = op.call(grads[0], s[0], s[1], s[2], s[3], s[4], s[5], s[6], s[7], s[8], s[9], s[10], s[11], s[12], s[13],
                     s[14], ctx->saved_data["top_k"].toInt(), n0, n2 || n3 || n4);
    out[0] = keep(std::get<0>(r), n0);
    if (n1) out[1] = std::get<4>(r).to(s[1].scalar_type());
    out[2] = keep(std::get<1>(r), n2);
    out[3] = keep(std::get<2>(r), n3);
    out[4] = keep(std::get<3>(r), n4);
    return out;
  }
};

std::tuple<Tensor, Tensor, Tensor> gather_experts_combine_autograd(
    const Tensor& x, const Tensor& weights, const Tensor& w1, const Tensor& w3, const Tensor& w2, const Tensor& tok,
    const Tensor& sor, const Tensor& ros, const Tensor& so, const Tensor& sc, const Tensor& te, const Tensor& tr,
    const Tensor& nt, int64_t K, int64_t cap, bool round_terms, bool save_gate_up) {
  if (!torch::autograd::compute_requires_grad(x, weights, w1, w3, w2)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<GecFwdSig>("mi355_moe::gather_experts_combine_fwd");
    return op.call(x, weights, w1, w3, w2, tok, sor, ros, so, sc, te, tr, nt, K, cap, round_terms, save_gate_up);
  }
  auto r = GatherExpertsCombine::apply(x, weights, w1, w3, w2, tok, sor, ros, so, sc, te, tr, nt, K, cap, round_terms,
                                       save_gate_up);
  return {r[0], r[1], r[2]};
}


// ---- selection with the (K+1)-th score: the same VJP, plain top-k ---------------------------------
using CutoffFwdSig = std::tuple<Tensor, Tensor, Tensor, Tensor>(const Tensor&, const OptTensor&, int64_t, int64_t,
                                                                 bool, double);

struct RouterSelectCutoff : public torch::autograd::Function<RouterSelectCutoff> {
  static variable_list forward(AutogradContext* ctx, const Tensor& logits, const OptTensor& bias, int64_t K,
                               int64_t score_func, bool route_norm, double route_scale) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<CutoffFwdSig>("mi355_moe::router_select_cutoff_fwd");
    auto r = op.call(logits, bias, K, score_func, route_norm, route_scale);
    ctx->save_for_backward({logits, std::get<1>(r)});
    ctx->saved_data["score_func"] = score_func;
    ctx->saved_data["route_norm"] = route_norm;
    ctx->saved_data["route_scale"] = route_scale;
    ctx->set_materialize_grads(false);  // no dense zero gradient for an unused score map
    ctx->mark_non_differentiable({std::get<1>(r)});
    return {std::get<0>(r), std::get<1>(r), std::get<2>(r), std::get<3>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(6);
    if (!ctx->needs_input_grad(0)) return out;
    const auto saved = ctx->get_saved_variables();
    static auto op = typed_op<SelectBwdSig>("mi355_moe::router_select_bwd");
    out[0] = op.call(saved[0], saved[1], opt(grads[0]), opt(grads[2]), ctx->saved_data["score_func"].toInt(),
                     ctx->saved_data["route_norm"].toBool(), ctx->saved_data["route_scale"].toDouble(),
                     /*mode: plain top-k*/ 0);
    return out;
  }
};

std::tuple<Tensor, Tensor, Tensor, Tensor> router_select_cutoff_autograd(const Tensor& logits, const OptTensor& bias,
                                                                         int64_t K, int64_t score_func, bool route_norm,
                                                                         double route_scale) {
  if (!torch::autograd::compute_requires_grad(logits)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<CutoffFwdSig>("mi355_moe::router_select_cutoff_fwd");
    return op.call(logits, bias, K, score_func, route_norm, route_scale);
  }
  auto r = RouterSelectCutoff::apply(logits, bias, K, score_func, route_norm, route_scale);
  return {r[0], r[1], r[2], r[3]};
}

// ---- RMS norm ---------------------------------------------------------------------------------------
using RmsFwdSig = std::tuple<Tensor, Tensor>(const Tensor&, const Tensor&, double);
using RmsBwdSig = std::tuple<Tensor, Tensor>(const Tensor&, const Tensor&, const Tensor&, const Tensor&, bool, bool);

struct RmsNorm : public torch::autograd::Function<RmsNorm> {
  static variable_list forward(AutogradContext* ctx, const Tensor& x, const Tensor& weight, double eps) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<RmsFwdSig>("mi355_moe::rms_norm_fwd");
    auto r = op.call(x, weight, eps);
    ctx->save_for_backward({x, weight, std::get<1>(r)});
    ctx->set_materialize_grads(false);
    return {std::get<0>(r), std::get<1>(r)};
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(3);
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1);
    if (!grads[0].defined() || !(n0 || n1)) return out;
    const auto s = ctx->get_saved_variables();
    static auto op = typed_op<RmsBwdSig>("mi355_moe::rms_norm_bwd");
    auto r = op.call(grads[0], s[0], s[1], s[2], n0, n1);
    out[0] = keep(std::get<0>(r), n0);
    out[1] = keep(std::get<1>(r), n1);
    return out;
  }
};

std::tuple<Tensor, Tensor> rms_norm_autograd(const Tensor& x, const Tensor& weight, double eps) {
  if (!torch::autograd::compute_requires_grad(x, weight)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<RmsFwdSig>("mi355_moe::rms_norm_fwd");
    return op.call(x, weight, eps);
  }
  auto r = RmsNorm::apply(x, weight, eps);
  return {r[0], r[1]};
}

// ---- load-balance loss: out = (loss, f_E...); the gradient flows into the scores -------------------
using BalanceFwdSig = Tensor(const Tensor&, const Tensor&, const OptTensor&);
using BalanceBwdSig = Tensor(const Tensor&, const Tensor&, const OptTensor&, const Tensor&);

struct BalanceLoss : public torch::autograd::Function<BalanceLoss> {
  static Tensor forward(AutogradContext* ctx, const Tensor& scores, const Tensor& map, const OptTensor& pad) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<BalanceFwdSig>("mi355_moe::balance_loss_fwd");
    Tensor out = op.call(scores, map, pad);
    ctx->save_for_backward({scores, out, pad.has_value() ? *pad : Tensor()});
    return out;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(3);
    if (!ctx->needs_input_grad(0) || !grads[0].defined()) return out;
    const auto s = ctx->get_saved_variables();
    static auto op = typed_op<BalanceBwdSig>("mi355_moe::balance_loss_bwd");
    out[0] = op.call(s[0], s[1].slice(0, 1), opt(s[2]), grads[0].slice(0, 0, 1));
    return out;
  }
};

Tensor balance_loss_autograd(const Tensor& scores, const Tensor& map, const OptTensor& pad) {
  if (!torch::autograd::compute_requires_grad(scores)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<BalanceFwdSig>("mi355_moe::balance_loss_fwd");
    return op.call(scores, map, pad);
  }
  return BalanceLoss::apply(scores, map, pad);
}

// ---- row gather: the backward sums the K row gradients of every token -----------------------------
using PermuteFwdSig = Tensor(const Tensor&, const Tensor&, const OptTensor&, const Tensor&, int64_t, int64_t);
using PermuteBwdSig = Tensor(const Tensor&, const Tensor&, int64_t, int64_t);

struct PermuteRows : public torch::autograd::Function<PermuteRows> {
  static Tensor forward(AutogradContext* ctx, const Tensor& x, const Tensor& ros, const OptTensor& sor,
                        const Tensor& total, int64_t K, int64_t cap) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<PermuteFwdSig>("mi355_moe::permute_rows_fwd");
    Tensor rows = op.call(x, ros, sor, total, K, cap);
    ctx->save_for_backward({ros});
    ctx->saved_data["num_tokens"] = x.size(0);
    ctx->saved_data["top_k"] = K;
    return rows;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(6);
    if (!ctx->needs_input_grad(0) || !grads[0].defined()) return out;
    const auto s = ctx->get_saved_variables();
    static auto op = typed_op<PermuteBwdSig>("mi355_moe::permute_rows_bwd");
    out[0] = op.call(grads[0], s[0], ctx->saved_data["num_tokens"].toInt(), ctx->saved_data["top_k"].toInt());
    return out;
  }
};

Tensor permute_rows_autograd(const Tensor& x, const Tensor& ros, const OptTensor& sor, const Tensor& total, int64_t K,
                             int64_t cap) {
  if (!torch::autograd::compute_requires_grad(x)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<PermuteFwdSig>("mi355_moe::permute_rows_fwd");
    return op.call(x, ros, sor, total, K, cap);
  }
  return PermuteRows::apply(x, ros, sor, total, K, cap);
}

// ---- combine: dY = weights * dout per row, dWeights = <y row, dout row> -----------------------------
using CombineFwdSig = Tensor(const Tensor&, const Tensor&, const Tensor&, const OptTensor&, const OptTensor&, int64_t,
                             int64_t, bool);
using CombineBwdSig = std::tuple<Tensor, Tensor>(const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                                                 const OptTensor&, const OptTensor&, int64_t);

struct Combine : public torch::autograd::Function<Combine> {
  static Tensor forward(AutogradContext* ctx, const Tensor& y, const Tensor& weights, const Tensor& ros,
                        const OptTensor& sor, const OptTensor& total, int64_t T, int64_t K, bool round_terms) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<CombineFwdSig>("mi355_moe::combine_fwd");
    Tensor out = op.call(y, weights, ros, sor, total, T, K, round_terms);
    ctx->save_for_backward({y, weights, ros, sor.has_value() ? *sor : Tensor(), total.has_value() ? *total : Tensor()});
    ctx->saved_data["top_k"] = K;
    return out;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(8);
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1);
    if (!grads[0].defined() || !(n0 || n1)) return out;
    const auto s = ctx->get_saved_variables();
    static auto op = typed_op<CombineBwdSig>("mi355_moe::combine_bwd");
    auto r = op.call(grads[0], s[0], s[1], s[2], opt(s[3]), opt(s[4]), ctx->saved_data["top_k"].toInt());
    out[0] = keep(std::get<0>(r), n0);
    if (n1) out[1] = std::get<1>(r).to(s[1].scalar_type());
    return out;
  }
};

Tensor combine_autograd(const Tensor& y, const Tensor& weights, const Tensor& ros, const OptTensor& sor,
                        const OptTensor& total, int64_t T, int64_t K, bool round_terms) {
  if (!torch::autograd::compute_requires_grad(y, weights)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<CombineFwdSig>("mi355_moe::combine_fwd");
    return op.call(y, weights, ros, sor, total, T, K, round_terms);
  }
  return Combine::apply(y, weights, ros, sor, total, T, K, round_terms);
}

// ---- one grouped linear map (the reference's GroupedExperts._grouped_mm) ----------------------------
using LinearFwdSig = Tensor(const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                            const Tensor&, bool);
using LinearBwdSig = std::tuple<Tensor, Tensor>(const Tensor&, const Tensor&, const Tensor&, const Tensor&,
                                                const Tensor&, const Tensor&, const Tensor&, const Tensor&, bool, bool,
                                                bool);

struct GroupedLinear : public torch::autograd::Function<GroupedLinear> {
  static Tensor forward(AutogradContext* ctx, const Tensor& x, const Tensor& w, const Tensor& so, const Tensor& sc,
                        const Tensor& te, const Tensor& tr, const Tensor& nt, bool zero_fill) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<LinearFwdSig>("mi355_moe::grouped_linear_fwd");
    Tensor y = op.call(x, w, so, sc, te, tr, nt, zero_fill);
    ctx->save_for_backward({x, w, so, sc, te, tr, nt});
    ctx->saved_data["zero_fill"] = zero_fill;
    ctx->set_materialize_grads(false);
    return y;
  }
  static variable_list backward(AutogradContext* ctx, variable_list grads) {
    variable_list out(8);
    const bool n0 = ctx->needs_input_grad(0), n1 = ctx->needs_input_grad(1);
    if (!grads[0].defined() || !(n0 || n1)) return out;
    const auto s = ctx->get_saved_variables();
    static auto op = typed_op<LinearBwdSig>("mi355_moe::grouped_linear_bwd");
    auto r = op.call(grads[0], s[0], s[1], s[2], s[3], s[4], s[5], s[6], n0, n1, ctx->saved_data["zero_fill"].toBool());
    out[0] = keep(std::get<0>(r), n0);
    out[1] = keep(std::get<1>(r), n1);
    return out;
  }
};

Tensor grouped_linear_autograd(const Tensor& x, const Tensor& w, const Tensor& so, const Tensor& sc, const Tensor& te,
                               const Tensor& tr, const Tensor& nt, bool zero_fill) {
  if (!torch::autograd::compute_requires_grad(x, w)) {
    at::AutoDispatchBelowADInplaceOrView below;
    static auto op = typed_op<LinearFwdSig>("mi355_moe::grouped_linear_fwd");
    return op.call(x, w, so, sc, te, tr, nt, zero_fill);
  }
  return GroupedLinear::apply(x, w, so, sc, te, tr, nt, zero_fill);
}

}  // namespace

TORCH_LIBRARY_IMPL(mi355_moe, Autograd, m) {
  m.impl("router_gate_fwd", router_gate_autograd);
  m.impl("router_select_fwd", router_select_autograd);
  m.impl("router_select_cutoff_fwd", router_select_cutoff_autograd);
  m.impl("rms_norm_fwd", rms_norm_autograd);
  m.impl("balance_loss_fwd", balance_loss_autograd);
  m.impl("permute_rows_fwd", permute_rows_autograd);
  m.impl("combine_fwd", combine_autograd);
  m.impl("grouped_linear_fwd", grouped_linear_autograd);
  m.impl("grouped_swiglu_fwd", grouped_swiglu_autograd);
  m.impl("rows_experts_combine_fwd", rows_experts_combine_autograd);
  m.impl("gather_experts_combine_fwd", gather_experts_combine_autograd);
}
