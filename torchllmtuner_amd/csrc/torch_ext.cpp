// torch.library registration of the MI355X MoE kernels: the `mi355_moe` operator namespace.
//
// A thin layer over the C ABI of include/mi355_moe.h.  Every operator takes and returns
// at::Tensor, allocates its outputs and workspaces through PyTorch's caching allocator,
// launches on the current HIP stream of its first tensor's device, never synchronises the
// host, and turns a negative return code into a Python exception (MI355_EINVAL ->
// ValueError, anything else -> RuntimeError) carrying mi355_moe_last_error().  Nothing is
// computed here: argument validation that mirrors the reference's messages lives in the
// Python host layer, shape propagation for tracing (fake tensors) in torchllmtuner_amd/ops.py,
// the autograd formulas there and in torch_autograd.cpp, and the arithmetic in the HIP kernels
// behind the C ABI.
//
// Plan tensors.  A permutation plan travels as plain int32 tensors: `small` packs
// counts_E (E) | seg_offsets (El+1) | seg_counts (El) | expert_order (El) |
// tile_expert (tile_cap) | tile_row0 (tile_cap) | num_tiles (1) in one allocation;
// seg_counts and expert_order must stay adjacent (the weight-gradient kernels read the
// experts' order right behind the counts).
#include <ATen/ATen.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>
#include <c10/core/DeviceGuard.h>
#include <torch/library.h>

#include <hip/hip_runtime_api.h>

#include <mutex>
#include <optional>
#include <tuple>

#include "../../include/mi355_moe.h"

namespace {

// A second stream per device (default priority, not synchronising with the null stream) and the
// two events of a fork / join around it.  The backward's weight gradients do not depend on its
// input gradient: launched there, their workgroups fill the CUs that the last, partly filled
// round of the other product's tiles leaves idle, and the bandwidth-bound row sum runs beside
// matrix work instead of between two launches.  Created on first use; never under stream
// capture (a caller who captures first runs a step uncaptured, as for every lazily built state);
// nullptr means "stay on one stream".
struct SideStream {
  hipStream_t stream = nullptr;
  hipEvent_t fork = nullptr, join = nullptr;
  std::mutex order;  // an event is recorded and waited for as one step: host threads share the pair

  // `to` waits for everything enqueued on `from` so far
  bool chain(hipEvent_t event, hipStream_t from, hipStream_t to) {
    std::lock_guard<std::mutex> lock(order);
    return hipEventRecord(event, from) == hipSuccess && hipStreamWaitEvent(to, event, 0) == hipSuccess;
  }
};

// which: 0 the weight gradients of the fused backward, 1 the shared expert (handed to the Python
// layer as a raw pointer, see aux_stream below)
SideStream* side_stream(int device, hipStream_t current, int which = 0) {
  static std::mutex mu;
  static SideStream streams[2][64];
  static bool attempted[2][64];
  if (device < 0 || device >= 64 || which < 0 || which > 1) return nullptr;
  std::lock_guard<std::mutex> lock(mu);
  SideStream& s = streams[which][device];
  bool* tried = attempted[which];
  if (!tried[device]) {
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(current, &capturing) != hipSuccess || capturing != hipStreamCaptureStatusNone)
      return nullptr;  // not now: try again on a later, uncaptured call
    tried[device] = true;
    if (hipStreamCreateWithFlags(&s.stream, hipStreamNonBlocking) != hipSuccess ||
        hipEventCreateWithFlags(&s.fork, hipEventDisableTiming) != hipSuccess ||
        hipEventCreateWithFlags(&s.join, hipEventDisableTiming) != hipSuccess) {
      (void)hipGetLastError();
      s.stream = nullptr;
    }
  }
  return s.stream ? &s : nullptr;
}

using at::Tensor;
using OptTensor = std::optional<Tensor>;

int dtype_code(const Tensor& t) {
  if (t.scalar_type() == at::kFloat) return MI355_F32;
  if (t.scalar_type() == at::kBFloat16) return MI355_BF16;
  if (t.scalar_type() == at::kDouble) return MI355_F64;
  TORCH_CHECK_TYPE(false, "MI355 MoE kernels support float32, bfloat16 and float64, got ", t.scalar_type());
}

void* ptr(const Tensor& t) { return (t.defined() && t.numel() > 0) ? t.data_ptr() : nullptr; }
void* ptr(const OptTensor& t) { return t.has_value() ? ptr(*t) : nullptr; }
const int32_t* iptr(const Tensor& t) { return static_cast<const int32_t*>(ptr(t)); }
const int32_t* iptr(const OptTensor& t) { return static_cast<const int32_t*>(ptr(t)); }
const float* fptr(const Tensor& t) { return static_cast<const float*>(ptr(t)); }
const float* fptr(const OptTensor& t) { return static_cast<const float*>(ptr(t)); }

// Device guard + the current stream of that device, for the duration of one operator.
struct Launch {
  c10::DeviceGuard guard;
  void* stream;
  explicit Launch(const Tensor& t)
      : guard(t.device()),
        stream(c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream()) {
    TORCH_CHECK(t.is_cuda(), "MI355 MoE kernels need tensors on a HIP device (got ", t.device(),
                "); there is no CPU implementation");
  }
};

void check(int rc, const char* what) {
  if (rc == MI355_OK) return;
  const char* msg = mi355_moe_last_error();
  TORCH_CHECK_VALUE(rc != MI355_EINVAL, what, " failed (", rc, "): ", msg);
  TORCH_CHECK(false, what, " failed (", rc, "): ", msg);
}

Tensor cf(const Tensor& t) { return t.scalar_type() == at::kFloat ? t.contiguous() : t.to(at::kFloat).contiguous(); }
Tensor bytes(int64_t n, const Tensor& like) {
  return at::empty({n > 0 ? n : 1}, like.options().dtype(at::kByte));
}
Tensor none_like(const Tensor& like) { return at::empty({0}, like.options()); }

// ------------------------------------------------------------------ router
Tensor router_gate_fwd(const Tensor& x_, const Tensor& w_, const OptTensor& bias_) {
  Launch L(x_);
  const Tensor x = x_.contiguous(), w = w_.contiguous();
  TORCH_CHECK_VALUE(x.dim() == 2 && w.dim() == 2 && w.size(1) == x.size(1), "gate weight ", w.sizes(),
                    " does not match input ", x.sizes());
  const int64_t T = x.size(0), D = x.size(1), E = w.size(0);
  OptTensor bias;
  if (bias_.has_value()) bias = cf(*bias_);
  Tensor out = at::empty({T, E}, x.options().dtype(at::kFloat));
  const int64_t nbytes = mi355_router_gate_fwd_workspace_bytes(T, D, E);
  Tensor ws;
  if (nbytes > 0) ws = bytes(nbytes, x);
  check(mi355_router_gate_fwd(ptr(x), dtype_code(x), ptr(w), dtype_code(w), fptr(bias), out.data_ptr<float>(),
                              ptr(ws), T, D, E, L.stream),
        "router_gate_fwd");
  return out;
}

std::tuple<Tensor, Tensor> router_gate_bwd(const Tensor& dlogits_, const Tensor& x_, const Tensor& w_, bool need_dx,
                                           bool need_dw) {
  Launch L(x_);
  const Tensor dl = cf(dlogits_), x = x_.contiguous(), w = w_.contiguous();
  const int64_t T = x.size(0), D = x.size(1), E = w.size(0);
  Tensor dx = need_dx ? at::empty_like(x) : none_like(x);
  Tensor dw = need_dw ? at::empty_like(w) : none_like(w);
  const int64_t nbytes = mi355_router_gate_bwd_workspace_bytes(T, D, E);
  Tensor ws;
  if (nbytes > 0) ws = bytes(nbytes, x);
  check(mi355_router_gate_bwd(fptr(dl), ptr(x), dtype_code(x), ptr(w), dtype_code(w), need_dx ? ptr(dx) : nullptr,
                              need_dw ? ptr(dw) : nullptr, ptr(ws), T, D, E, L.stream),
        "router_gate_bwd");
  return {dx, dw};
}

std::tuple<Tensor, Tensor, Tensor, Tensor> router_select_fwd(const Tensor& logits_, const OptTensor& bias_,
                                                             int64_t K, int64_t score_func, bool route_norm,
                                                             double route_scale, int64_t num_groups,
                                                             int64_t num_limited, int64_t mode, bool want_scores,
                                                             bool want_map) {
  Launch L(logits_);
  TORCH_CHECK_TYPE(logits_.scalar_type() == at::kFloat, "router logits must be float32");
  const Tensor logits = logits_.contiguous();
  const int64_t T = logits.size(0), E = logits.size(1);
  OptTensor bias;
  if (bias_.has_value()) bias = cf(*bias_);
  Tensor weights = at::empty({T, K}, logits.options());
  Tensor ids = at::empty({T, K}, logits.options().dtype(at::kLong));
  Tensor scores = want_scores ? at::empty({T, E}, logits.options()) : none_like(logits);
  Tensor map = at::empty({want_map ? T : 0, want_map ? E : 0}, logits.options().dtype(at::kBool));
  check(mi355_router_select_fwd(fptr(logits), fptr(bias), weights.data_ptr<float>(), ids.data_ptr<int64_t>(),
                                want_scores ? scores.data_ptr<float>() : nullptr,
                                want_map ? static_cast<uint8_t*>(ptr(map)) : nullptr, T, E, K, (int)score_func,
                                (int)route_norm, (float)route_scale, (int)num_groups, (int)num_limited, (int)mode,
                                L.stream),
        "router_select_fwd");
  return {weights, ids, scores, map};
}

std::tuple<Tensor, Tensor, Tensor, Tensor> router_select_cutoff_fwd(const Tensor& logits_, const OptTensor& bias_,
                                                                    int64_t K, int64_t score_func, bool route_norm,
                                                                    double route_scale) {
  Launch L(logits_);
  TORCH_CHECK_TYPE(logits_.scalar_type() == at::kFloat, "router logits must be float32");
  const Tensor logits = logits_.contiguous();
  const int64_t T = logits.size(0), E = logits.size(1);
  OptTensor bias;
  if (bias_.has_value()) bias = cf(*bias_);
  Tensor weights = at::empty({T, K}, logits.options());
  Tensor ids = at::empty({T, K}, logits.options().dtype(at::kLong));
  Tensor scores = at::empty({T, E}, logits.options());
  Tensor cutoff = at::empty({T}, logits.options());
  check(mi355_router_select_cutoff_fwd(fptr(logits), fptr(bias), weights.data_ptr<float>(), ids.data_ptr<int64_t>(),
                                       scores.data_ptr<float>(), cutoff.data_ptr<float>(), T, E, K, (int)score_func,
                                       (int)route_norm, (float)route_scale, L.stream),
        "router_select_cutoff_fwd");
  return {weights, ids, scores, cutoff};
}

Tensor router_select_bwd(const Tensor& logits_, const Tensor& ids_, const OptTensor& dweights_,
                         const OptTensor& dscores_, int64_t score_func, bool route_norm, double route_scale,
                         int64_t mode) {
  Launch L(logits_);
  const Tensor logits = logits_.contiguous(), ids = ids_.contiguous();
  const int64_t T = logits.size(0), E = logits.size(1), K = ids.size(1);
  OptTensor dw, ds;
  if (dweights_.has_value()) dw = cf(*dweights_);
  if (dscores_.has_value()) ds = cf(*dscores_);
  Tensor out = at::empty_like(logits);
  check(mi355_router_select_bwd(fptr(logits), static_cast<const int64_t*>(ptr(ids)), fptr(dw), fptr(ds),
                                out.data_ptr<float>(), T, E, K, (int)score_func, (int)route_norm,
                                (float)route_scale, (int)mode, L.stream),
        "router_select_bwd");
  return out;
}

void quantile_observe(Tensor histogram, const Tensor& scores_, const Tensor& cutoff_, const Tensor& bias_,
                      const OptTensor& pad_) {
  Launch L(histogram);
  TORCH_CHECK_TYPE(histogram.scalar_type() == at::kLong && histogram.is_contiguous(),
                   "histogram_EB must be a contiguous int64 tensor");
  const Tensor scores = cf(scores_), cutoff = cf(cutoff_.reshape({-1})), bias = cf(bias_);
  const int64_t T = scores.size(0), E = scores.size(1);
  OptTensor pad;
  if (pad_.has_value()) pad = pad_->contiguous();
  check(mi355_quantile_observe(fptr(scores), fptr(cutoff), fptr(bias), static_cast<const uint8_t*>(ptr(pad)),
                               histogram.data_ptr<int64_t>(), T, E, histogram.size(1), L.stream),
        "quantile_observe");
}

Tensor quantile_estimate(const Tensor& histogram_, const Tensor& bias_, int64_t K) {
  Launch L(histogram_);
  TORCH_CHECK_TYPE(histogram_.scalar_type() == at::kLong, "histogram_EB must be int64");
  const Tensor hist = histogram_.contiguous(), bias = cf(bias_);
  const int64_t E = hist.size(0), B = hist.size(1);
  Tensor out = at::empty({E}, bias.options());
  Tensor ws = at::empty({2 * E}, bias.options());
  check(mi355_quantile_estimate(static_cast<const int64_t*>(ptr(hist)), fptr(bias), out.data_ptr<float>(), ptr(ws), E,
                                K, B, L.stream),
        "quantile_estimate");
  return out;
}

std::tuple<Tensor, Tensor> rms_norm_fwd(const Tensor& x_, const Tensor& weight_, double eps) {
  Launch L(x_);
  TORCH_CHECK_TYPE(x_.scalar_type() == weight_.scalar_type(), "rms_norm: input (", x_.scalar_type(), ") and weight (",
                   weight_.scalar_type(), ") must share a dtype");
  const Tensor x = x_.contiguous(), weight = weight_.contiguous();
  const int64_t D = weight.numel(), rows = D > 0 ? x.numel() / D : 0;
  Tensor y = at::empty_like(x);
  Tensor rstd = at::empty({rows}, x.options().dtype(at::kFloat));
  check(mi355_rms_norm_fwd(ptr(x), ptr(weight), dtype_code(x), ptr(y), static_cast<float*>(ptr(rstd)), rows, D,
                           (float)eps, L.stream),
        "rms_norm_fwd");
  return {y, rstd};
}

std::tuple<Tensor, Tensor> rms_norm_bwd(const Tensor& dy_, const Tensor& x_, const Tensor& weight_,
                                        const Tensor& rstd, bool need_dx, bool need_dw) {
  Launch L(x_);
  const Tensor x = x_.contiguous(), weight = weight_.contiguous();
  const Tensor dy = (dy_.scalar_type() == x.scalar_type() ? dy_ : dy_.to(x.scalar_type())).contiguous();
  const int64_t D = weight.numel(), rows = D > 0 ? x.numel() / D : 0;
  Tensor dx = need_dx ? at::empty_like(x) : none_like(x);
  Tensor dw = need_dw ? at::empty_like(weight) : none_like(weight);
  Tensor ws;
  if (need_dw) ws = bytes(mi355_rms_norm_bwd_workspace_bytes(rows, D), x);
  check(mi355_rms_norm_bwd(ptr(dy), ptr(x), ptr(weight), fptr(rstd), dtype_code(x), need_dx ? ptr(dx) : nullptr,
                           need_dw ? ptr(dw) : nullptr, ptr(ws), rows, D, L.stream),
        "rms_norm_bwd");
  return {dx, dw};
}

Tensor balance_loss_fwd(const Tensor& scores_, const Tensor& map_, const OptTensor& pad_) {
  Launch L(scores_);
  TORCH_CHECK_TYPE(scores_.scalar_type() == at::kFloat, "router scores must be float32");
  const Tensor scores = scores_.contiguous(), map = map_.contiguous();
  const int64_t T = scores.size(0), E = scores.size(1);
  OptTensor pad;
  if (pad_.has_value()) pad = pad_->contiguous();
  Tensor out = at::empty({1 + E}, scores.options());
  Tensor ws = bytes(mi355_balance_loss_workspace_bytes(T, E), scores);
  check(mi355_balance_loss_fwd(fptr(scores), static_cast<const uint8_t*>(ptr(map)),
                               static_cast<const uint8_t*>(ptr(pad)), out.data_ptr<float>(),
                               out.data_ptr<float>() + 1, ptr(ws), T, E, L.stream),
        "balance_loss_fwd");
  return out;
}

Tensor balance_loss_bwd(const Tensor& scores_, const Tensor& f_, const OptTensor& pad_, const Tensor& grad_) {
  Launch L(scores_);
  const Tensor scores = scores_.contiguous(), f = cf(f_), g = cf(grad_.reshape({1}));
  const int64_t T = scores.size(0), E = scores.size(1);
  OptTensor pad;
  if (pad_.has_value()) pad = pad_->contiguous();
  Tensor out = at::empty_like(scores);
  check(mi355_balance_loss_bwd(fptr(scores), fptr(f), static_cast<const uint8_t*>(ptr(pad)), fptr(g),
                               out.data_ptr<float>(), T, E, L.stream),
        "balance_loss_bwd");
  return out;
}

// ------------------------------------------------------------------ plan
int64_t tile_m() { return mi355_grouped_tile_m(MI355_BF16); }

std::tuple<Tensor, Tensor, Tensor> permute_plan(const Tensor& ids_, int64_t E, int64_t lo, int64_t hi, int64_t align) {
  Launch L(ids_);
  const Tensor ids = (ids_.scalar_type() == at::kLong ? ids_ : ids_.to(at::kLong)).contiguous();
  TORCH_CHECK_VALUE(ids.dim() == 2, "expert ids must have shape (tokens, top_k)");
  const int64_t T = ids.size(0), K = ids.size(1), N = T * K, El = hi - lo, tm = tile_m();
  TORCH_CHECK_VALUE(El >= 1, "permute_plan: empty local expert range");
  const int64_t row_cap = N + (align > 1 ? El * (align - 1) : 0);
  const int64_t tile_cap = N / tm + El + 1;
  const auto i32 = ids.options().dtype(at::kInt);
  Tensor small = at::empty({E + (El + 1) + 2 * El + 2 * tile_cap + 1}, i32);
  int32_t* p = small.data_ptr<int32_t>();
  int32_t* counts_E = p; p += E;
  int32_t* seg_offsets = p; p += El + 1;
  int32_t* seg_counts = p; p += 2 * El;
  int32_t* tile_expert = p; p += tile_cap;
  int32_t* tile_row0 = p; p += tile_cap;
  int32_t* num_tiles = p;
  Tensor row_of_slot = at::empty({N}, i32);
  Tensor rows2 = at::empty({2, row_cap}, i32);
  Tensor ws = bytes(mi355_permute_plan_workspace_bytes(T, K, E), ids);
  check(mi355_permute_plan(static_cast<const int64_t*>(ptr(ids)), T, K, E, lo, hi, align, tm, counts_E, seg_offsets,
                           seg_counts, static_cast<int32_t*>(ptr(row_of_slot)),
                           row_cap > 0 ? rows2.data_ptr<int32_t>() : nullptr,
                           row_cap > 0 ? rows2.data_ptr<int32_t>() + row_cap : nullptr, row_cap, tile_expert,
                           tile_row0, num_tiles, tile_cap, ptr(ws), L.stream),
        "permute_plan");
  return {small, row_of_slot, rows2};
}

Tensor segments_from_counts(const Tensor& counts_, int64_t total_rows) {
  Launch L(counts_);
  const Tensor counts = (counts_.scalar_type() == at::kInt ? counts_ : counts_.to(at::kInt)).contiguous();
  const int64_t El = counts.size(0), tm = tile_m();
  const int64_t tile_cap = total_rows / tm + El + 1;
  Tensor small = at::empty({(El + 1) + 2 * El + 2 * tile_cap + 1}, counts.options());
  int32_t* p = small.data_ptr<int32_t>();
  int32_t* seg_offsets = p; p += El + 1;
  int32_t* seg_counts = p; p += 2 * El;
  int32_t* tile_expert = p; p += tile_cap;
  int32_t* tile_row0 = p; p += tile_cap;
  int32_t* num_tiles = p;
  check(mi355_segments_from_counts(iptr(counts), El, tm, total_rows, seg_offsets, seg_counts, tile_expert, tile_row0,
                                   num_tiles, tile_cap, L.stream),
        "segments_from_counts");
  return small;
}

// ------------------------------------------------------------------ row movers, combine
Tensor permute_rows_fwd(const Tensor& x_, const Tensor& row_of_slot, const OptTensor& slot_of_row,
                        const Tensor& total_rows, int64_t K, int64_t row_capacity) {
  Launch L(x_);
  const Tensor x = x_.contiguous();
  const int64_t T = x.size(0), D = x.size(1);
  Tensor rows = at::empty({row_capacity, D}, x.options());
  check(mi355_permute_rows_fwd(ptr(x), dtype_code(x), iptr(row_of_slot), iptr(slot_of_row), iptr(total_rows),
                               ptr(rows), T, D, K, row_capacity, L.stream),
        "permute_rows_fwd");
  return rows;
}

Tensor permute_rows_bwd(const Tensor& drows_, const Tensor& row_of_slot, int64_t T, int64_t K) {
  Launch L(drows_);
  const Tensor drows = drows_.contiguous();
  const int64_t D = drows.size(1);
  Tensor dx = at::empty({T, D}, drows.options());
  check(mi355_permute_rows_bwd(ptr(drows), dtype_code(drows), iptr(row_of_slot), ptr(dx), T, D, K, L.stream),
        "permute_rows_bwd");
  return dx;
}

// slot_of_row / total_rows are not read here: they ride along for the backward (autograd saves
// the operator's inputs), which zeroes the gradient of a padded plan's padding rows
Tensor combine_fwd(const Tensor& y_, const Tensor& weights_, const Tensor& row_of_slot, const OptTensor& slot_of_row,
                   const OptTensor& total_rows, int64_t T, int64_t K, bool round_terms) {
  (void)slot_of_row;
  (void)total_rows;
  Launch L(y_);
  const Tensor y = y_.contiguous(), w = cf(weights_);
  const int64_t D = y.size(1);
  Tensor out = at::empty({T, D}, y.options());
  check(mi355_combine_fwd(ptr(y), dtype_code(y), fptr(w), iptr(row_of_slot), ptr(out), T, D, K, (int)round_terms,
                          L.stream),
        "combine_fwd");
  return out;
}

std::tuple<Tensor, Tensor> combine_bwd(const Tensor& dout_, const Tensor& y_, const Tensor& weights_,
                                       const Tensor& row_of_slot, const OptTensor& slot_of_row,
                                       const OptTensor& total_rows, int64_t K) {
  Launch L(y_);
  const Tensor y = y_.contiguous(), w = cf(weights_);
  const Tensor dout = (dout_.scalar_type() == y.scalar_type() ? dout_ : dout_.to(y.scalar_type())).contiguous();
  const int64_t T = dout.size(0), D = y.size(1), R = y.size(0);
  Tensor dy = at::empty_like(y);
  Tensor dw = at::empty({T, K}, y.options().dtype(at::kFloat));
  check(mi355_combine_bwd(ptr(dout), ptr(y), dtype_code(y), fptr(w), iptr(row_of_slot), iptr(slot_of_row),
                          iptr(total_rows), ptr(dy), static_cast<float*>(ptr(dw)), T, D, K, R, L.stream),
        "combine_bwd");
  return {dy, dw};
}

Tensor combine_row_scale(const Tensor& weights_, const Tensor& slot_of_row, int64_t row_capacity) {
  Launch L(weights_);
  const Tensor w = cf(weights_);
  const int64_t T = w.size(0), K = w.size(1);
  Tensor out = at::empty({row_capacity}, w.options());
  check(mi355_combine_row_scale(fptr(w), iptr(slot_of_row), static_cast<float*>(ptr(out)), T, K, row_capacity,
                                L.stream),
        "combine_row_scale");
  return out;
}

Tensor combine_scores_bwd(const Tensor& partial, const Tensor& row_of_slot, int64_t T, int64_t K) {
  Launch L(partial);
  Tensor dw = at::empty({T, K}, partial.options());
  check(mi355_combine_scores_bwd(fptr(partial), partial.size(1), iptr(row_of_slot), static_cast<float*>(ptr(dw)), T,
                                 K, partial.size(0), L.stream),
        "combine_scores_bwd");
  return dw;
}

// ------------------------------------------------------------------ experts
struct Plan {
  const int32_t *seg_offsets, *seg_counts, *tile_expert, *tile_row0, *num_tiles;
  int64_t tile_capacity;
};
Plan plan_of(const Tensor& seg_offsets, const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0,
             const Tensor& num_tiles) {
  return {iptr(seg_offsets), iptr(seg_counts), iptr(tile_expert), iptr(tile_row0), iptr(num_tiles),
          tile_expert.numel()};
}

void check_weights(const Tensor& rows, const Tensor& w1, const Tensor& w3, const Tensor& w2) {
  TORCH_CHECK_VALUE(w1.dim() == 3 && w1.size(2) == rows.size(1) && w3.sizes() == w1.sizes() && w2.dim() == 3 &&
                        w2.size(0) == w1.size(0) && w2.size(1) == w1.size(2) && w2.size(2) == w1.size(1),
                    "expert weight shapes do not match (E,F,D)/(E,F,D)/(E,D,F)");
  TORCH_CHECK_TYPE(w1.scalar_type() == rows.scalar_type() && w3.scalar_type() == rows.scalar_type() &&
                       w2.scalar_type() == rows.scalar_type(),
                   "expert weights and rows must share one dtype");
}

// zero_fill: rows that the plan does not cover come back as zeros instead of uninitialised
// memory (for callers whose counts may not add up to the rows they pass)
std::tuple<Tensor, Tensor, Tensor, Tensor> grouped_swiglu_fwd(
    const Tensor& rows_, const OptTensor& token_of_row, const Tensor& w1_, const Tensor& w3_, const Tensor& w2_,
    const Tensor& seg_offsets, const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0,
    const Tensor& num_tiles, int64_t row_capacity, bool zero_fill) {
  Launch L(rows_);
  const Tensor rows = rows_.contiguous(), w1 = w1_.contiguous(), w3 = w3_.contiguous(), w2 = w2_.contiguous();
  check_weights(rows, w1, w3, w2);
  const int64_t D = rows.size(1), El = w1.size(0), F = w1.size(1), R = row_capacity;
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  Tensor gate = at::empty({R, F}, rows.options()), up = at::empty({R, F}, rows.options());
  Tensor h = at::empty({R, F}, rows.options());
  Tensor y = zero_fill ? at::zeros({R, D}, rows.options()) : at::empty({R, D}, rows.options());
  check(mi355_grouped_swiglu_fwd(ptr(rows), iptr(token_of_row), rows.size(0), ptr(w1), ptr(w3), ptr(w2),
                                 dtype_code(rows), p.seg_offsets, p.seg_counts, p.tile_expert, p.tile_row0, p.num_tiles,
                                 p.tile_capacity, ptr(gate), ptr(up), ptr(h), ptr(y), El, D, F, R, L.stream),
        "grouped_swiglu_fwd");
  return {y, gate, up, h};
}

std::tuple<Tensor, Tensor, Tensor, Tensor> grouped_swiglu_bwd(
    const Tensor& dy_, const Tensor& rows_, const OptTensor& token_of_row, const Tensor& w1_, const Tensor& w3_,
    const Tensor& w2_, const Tensor& gate, const Tensor& up, const Tensor& h, const Tensor& seg_offsets,
    const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0, const Tensor& num_tiles,
    bool need_drows, bool need_dw, bool zero_fill) {
  Launch L(rows_);
  const Tensor rows = rows_.contiguous(), w1 = w1_.contiguous(), w3 = w3_.contiguous(), w2 = w2_.contiguous();
  const Tensor dy = (dy_.scalar_type() == rows.scalar_type() ? dy_ : dy_.to(rows.scalar_type())).contiguous();
  const int64_t D = rows.size(1), El = w1.size(0), F = w1.size(1), R = dy.size(0);
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  Tensor dgate = at::empty_like(gate), dup = at::empty_like(up);
  Tensor drows = !need_drows ? none_like(rows)
                             : (zero_fill ? at::zeros({R, D}, rows.options()) : at::empty({R, D}, rows.options()));
  Tensor dw1 = need_dw ? at::empty_like(w1) : none_like(w1);
  Tensor dw3 = need_dw ? at::empty_like(w3) : none_like(w3);
  Tensor dw2 = need_dw ? at::empty_like(w2) : none_like(w2);
  check(mi355_grouped_swiglu_bwd(ptr(dy), ptr(rows), iptr(token_of_row), rows.size(0), ptr(w1), ptr(w3), ptr(w2),
                                 ptr(gate), ptr(up), ptr(h), dtype_code(rows), p.seg_offsets, p.seg_counts,
                                 p.tile_expert, p.tile_row0, p.num_tiles, p.tile_capacity, ptr(dgate), ptr(dup),
                                 need_drows ? ptr(drows) : nullptr, need_dw ? ptr(dw1) : nullptr,
                                 need_dw ? ptr(dw3) : nullptr, need_dw ? ptr(dw2) : nullptr, El, D, F, R, L.stream),
        "grouped_swiglu_bwd");
  return {drows, dw1, dw3, dw2};
}

// y[r] = x[r] . w[e(r)]^T over the plan's segments (GroupedExperts._grouped_mm of the reference)
Tensor grouped_linear_fwd(const Tensor& x_, const Tensor& w_, const Tensor& seg_offsets, const Tensor& seg_counts,
                          const Tensor& tile_expert, const Tensor& tile_row0, const Tensor& num_tiles,
                          bool zero_fill) {
  Launch L(x_);
  const Tensor x = x_.contiguous(), w = w_.contiguous();
  TORCH_CHECK_VALUE(x.dim() == 2 && w.dim() == 3 && w.size(2) == x.size(1), "grouped weight ", w.sizes(),
                    " does not match rows ", x.sizes());
  TORCH_CHECK_TYPE(w.scalar_type() == x.scalar_type(), "grouped weight and rows must share one dtype");
  const int64_t R = x.size(0), I = x.size(1), El = w.size(0), O = w.size(1);
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  Tensor y = zero_fill ? at::zeros({R, O}, x.options()) : at::empty({R, O}, x.options());
  check(mi355_grouped_linear_fwd(ptr(x), ptr(w), dtype_code(x), p.seg_offsets, p.seg_counts, p.tile_expert,
                                 p.tile_row0, p.num_tiles, p.tile_capacity, ptr(y), El, I, O, R, L.stream),
        "grouped_linear_fwd");
  return y;
}

std::tuple<Tensor, Tensor> grouped_linear_bwd(const Tensor& dy_, const Tensor& x_, const Tensor& w_,
                                              const Tensor& seg_offsets, const Tensor& seg_counts,
                                              const Tensor& tile_expert, const Tensor& tile_row0,
                                              const Tensor& num_tiles, bool need_dx, bool need_dw, bool zero_fill) {
  Launch L(x_);
  const Tensor x = x_.contiguous(), w = w_.contiguous();
  const Tensor dy = (dy_.scalar_type() == x.scalar_type() ? dy_ : dy_.to(x.scalar_type())).contiguous();
  const int64_t R = x.size(0), I = x.size(1), El = w.size(0), O = w.size(1);
  TORCH_CHECK_VALUE(dy.dim() == 2 && dy.size(0) == R && dy.size(1) == O, "grouped_linear_bwd: gradient ", dy.sizes(),
                    " does not match (", R, ", ", O, ")");
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  Tensor dx = !need_dx ? none_like(x) : (zero_fill ? at::zeros({R, I}, x.options()) : at::empty({R, I}, x.options()));
  Tensor dw = need_dw ? at::empty_like(w) : none_like(w);
  check(mi355_grouped_linear_bwd(ptr(dy), ptr(x), ptr(w), dtype_code(x), p.seg_offsets, p.seg_counts, p.tile_expert,
                                 p.tile_row0, p.num_tiles, p.tile_capacity, need_dx ? ptr(dx) : nullptr,
                                 need_dw ? ptr(dw) : nullptr, El, I, O, R, L.stream),
        "grouped_linear_bwd");
  return {dx, dw};
}

// out[t] = sum_k weights[t,k] * experts(x)[row(t,k)]: gathered expert product, then the combine.
// Returns (out, gate, up); y and h are dropped (the fused backward recomputes h).  save_gate_up = false
// (nobody will differentiate): gate and up are not written at all and come back empty.
std::tuple<Tensor, Tensor, Tensor> gather_experts_combine_fwd(
    const Tensor& x_, const Tensor& weights_, const Tensor& w1_, const Tensor& w3_, const Tensor& w2_,
    const Tensor& token_of_row, const Tensor& slot_of_row, const Tensor& row_of_slot, const Tensor& seg_offsets,
    const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0, const Tensor& num_tiles, int64_t K,
    int64_t row_capacity, bool round_terms, bool save_gate_up) {
  (void)slot_of_row;  // for the backward only (the row -> slot index behind the row scales)
  Launch L(x_);
  const Tensor x = x_.contiguous(), w1 = w1_.contiguous(), w3 = w3_.contiguous(), w2 = w2_.contiguous();
  check_weights(x, w1, w3, w2);
  const Tensor w = cf(weights_);
  const int64_t T = x.size(0), D = x.size(1), El = w1.size(0), F = w1.size(1), R = row_capacity;
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  const int64_t Rs = save_gate_up ? R : 0;
  Tensor gate = at::empty({Rs, F}, x.options()), up = at::empty({Rs, F}, x.options());
  Tensor h = at::empty({R, F}, x.options()), y = at::empty({R, D}, x.options());
  check(mi355_grouped_swiglu_fwd(ptr(x), iptr(token_of_row), T, ptr(w1), ptr(w3), ptr(w2), dtype_code(x),
                                 p.seg_offsets, p.seg_counts, p.tile_expert, p.tile_row0, p.num_tiles,
                                 p.tile_capacity, save_gate_up ? ptr(gate) : nullptr, save_gate_up ? ptr(up) : nullptr, ptr(h),
                                 ptr(y), El, D, F, R, L.stream),
        "grouped_swiglu_fwd");
  Tensor out = at::empty({T, D}, x.options());
  check(mi355_combine_fwd(ptr(y), dtype_code(y), fptr(w), iptr(row_of_slot), ptr(out), T, D, K, (int)round_terms,
                          L.stream),
        "combine_fwd");
  return {out, gate, up};
}

// Backward of the above in one pass (mi355_grouped_swiglu_combine_bwd): the K-way row sum
// that turns the expert-major input gradient into dx runs right behind the kernel that wrote
// it, while those rows are still in the memory-side cache; the weight-gradient kernels follow.
// Returns (dx, dw1, dw3, dw2, dweights).
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor> gather_experts_combine_bwd(
    const Tensor& dout_, const Tensor& x_, const Tensor& weights_, const Tensor& w1_, const Tensor& w3_,
    const Tensor& w2_, const Tensor& gate, const Tensor& up, const Tensor& token_of_row, const Tensor& slot_of_row,
    const Tensor& row_of_slot, const Tensor& seg_offsets, const Tensor& seg_counts, const Tensor& tile_expert,
    const Tensor& tile_row0, const Tensor& num_tiles, int64_t K, bool need_dx, bool need_dw) {
  Launch L(x_);
  const Tensor x = x_.contiguous(), w1 = w1_.contiguous(), w3 = w3_.contiguous(), w2 = w2_.contiguous();
  const Tensor dout = (dout_.scalar_type() == x.scalar_type() ? dout_ : dout_.to(x.scalar_type())).contiguous();
  const Tensor w = cf(weights_);
  const int64_t T = x.size(0), D = x.size(1), El = w1.size(0), F = w1.size(1), R = gate.size(0);
  const int64_t slots = mi355_grouped_combine_bwd_slots(dtype_code(x), D, F);
  TORCH_CHECK(slots > 0, "gather_experts_combine_bwd does not cover this dtype/shape");
  const Plan p = plan_of(seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles);
  Tensor row_scale = at::empty({R}, w.options());
  check(mi355_combine_row_scale(fptr(w), iptr(slot_of_row), static_cast<float*>(ptr(row_scale)), T, K, R, L.stream),
        "combine_row_scale");
  Tensor dgate = at::empty_like(gate), dup = at::empty_like(up), hs = at::empty_like(gate);
  Tensor partial = at::empty({R, slots}, w.options());
  Tensor drows = need_dx ? at::empty({R, D}, x.options()) : none_like(x);
  Tensor dw1 = need_dw ? at::empty_like(w1) : none_like(w1);
  Tensor dw3 = need_dw ? at::empty_like(w3) : none_like(w3);
  Tensor dw2 = need_dw ? at::empty_like(w2) : none_like(w2);
  auto run = [&](int stages, void* stream) {
    check(mi355_grouped_swiglu_combine_bwd(
              ptr(dout), ptr(x), iptr(token_of_row), T, fptr(row_scale), ptr(w1), ptr(w3), ptr(w2), ptr(gate),
              ptr(up), dtype_code(x), p.seg_offsets, p.seg_counts, p.tile_expert, p.tile_row0, p.num_tiles,
              p.tile_capacity, ptr(dgate), ptr(dup), ptr(hs), static_cast<float*>(ptr(partial)),
              need_dx ? ptr(drows) : nullptr, need_dw ? ptr(dw1) : nullptr, need_dw ? ptr(dw3) : nullptr,
              need_dw ? ptr(dw2) : nullptr, El, D, F, R, stages, stream),
          "grouped_swiglu_combine_bwd");
  };
  Tensor dx = need_dx ? at::empty({T, D}, x.options()) : none_like(x);
  Tensor dweights = at::empty({T, K}, w.options());
  auto sums = [&]() {
    if (need_dx)
      check(mi355_permute_rows_bwd(ptr(drows), dtype_code(x), iptr(row_of_slot), ptr(dx), T, D, K, L.stream),
            "permute_rows_bwd");
    check(mi355_combine_scores_bwd(fptr(partial), slots, iptr(row_of_slot), static_cast<float*>(ptr(dweights)), T, K,
                                   R, L.stream),
          "combine_scores_bwd");
  };
  const hipStream_t main = static_cast<hipStream_t>(L.stream);
  SideStream* side = (R > 0 && need_dw && need_dx) ? side_stream(x.device().index(), main) : nullptr;
  if (R == 0) {
    run(0, L.stream);  // no rows: only the zero weight gradients remain to be written
    sums();
  } else if (!side) {
    run(MI355_STAGE_DH | (need_dx ? MI355_STAGE_DX : 0), L.stream);
    sums();
    if (need_dw) run(MI355_STAGE_DW2 | MI355_STAGE_DW1 | MI355_STAGE_DW3, L.stream);
  } else {
    // Everything after dH reads what dH wrote and nothing else of this call: the weight gradients
    // go to the side stream; the input gradient, its row sum and the score gradient stay here;
    // this stream waits for the other before the operator returns, so that whatever the caller
    // enqueues next, and the allocator's reuse of these buffers, is ordered behind both.
    run(MI355_STAGE_DH, L.stream);
    TORCH_CHECK(side->chain(side->fork, main, side->stream),
                "gather_experts_combine_bwd: cannot fork to the side stream: ", hipGetErrorString(hipGetLastError()));
    run(MI355_STAGE_DW2 | MI355_STAGE_DW1 | MI355_STAGE_DW3, side->stream);
    run(MI355_STAGE_DX, L.stream);
    sums();
    TORCH_CHECK(side->chain(side->join, side->stream, main),
                "gather_experts_combine_bwd: cannot join the side stream: ", hipGetErrorString(hipGetLastError()));
  }
  return {dx, dw1, dw3, dw2, dweights};
}

// The three stages of the routed path that has no folded form (fp32, fp64, shapes off the bf16
// MFMA path) as ONE operator each way: row scatter, grouped SwiGLU experts and combine going
// forward; combine, experts and K-way row sum going back.  Nothing new is computed -- these call
// the stage operators above in order -- but a step then crosses the dispatcher and the autograd
// engine once per direction instead of three times, which is what a small step's time is made of.
// Returns (out, rows, gate, up, h, y): everything but `out` is kept for the backward.
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor, Tensor> rows_experts_combine_fwd(
    const Tensor& x, const Tensor& weights, const Tensor& w1, const Tensor& w3, const Tensor& w2,
    const Tensor& row_of_slot, const OptTensor& slot_of_row, const Tensor& total_rows, const Tensor& seg_offsets,
    const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0, const Tensor& num_tiles, int64_t K,
    int64_t row_capacity, bool round_terms) {
  Tensor rows = permute_rows_fwd(x, row_of_slot, slot_of_row, total_rows, K, row_capacity);
  auto [y, gate, up, h] = grouped_swiglu_fwd(rows, std::nullopt, w1, w3, w2, seg_offsets, seg_counts, tile_expert,
                                             tile_row0, num_tiles, row_capacity, false);
  Tensor out = combine_fwd(y, weights, row_of_slot, slot_of_row, total_rows, x.size(0), K, round_terms);
  return {out, rows, gate, up, h, y};
}

// Returns (dx, dw1, dw3, dw2, dweights).
std::tuple<Tensor, Tensor, Tensor, Tensor, Tensor> rows_experts_combine_bwd(
    const Tensor& dout, const Tensor& rows, const Tensor& weights, const Tensor& w1, const Tensor& w3,
    const Tensor& w2, const Tensor& gate, const Tensor& up, const Tensor& h, const Tensor& y,
    const Tensor& row_of_slot, const OptTensor& slot_of_row, const Tensor& total_rows, const Tensor& seg_offsets,
    const Tensor& seg_counts, const Tensor& tile_expert, const Tensor& tile_row0, const Tensor& num_tiles, int64_t T,
    int64_t K, bool need_dx, bool need_dw) {
  auto [dy, dweights] = combine_bwd(dout, y, weights, row_of_slot, slot_of_row, total_rows, K);
  auto [drows, dw1, dw3, dw2] = grouped_swiglu_bwd(dy, rows, std::nullopt, w1, w3, w2, gate, up, h, seg_offsets,
                                                   seg_counts, tile_expert, tile_row0, num_tiles, need_dx, need_dw,
                                                   false);
  Tensor dx = need_dx ? permute_rows_bwd(drows, row_of_slot, T, K) : none_like(rows);
  return {dx, dw1, dw3, dw2, dweights};
}

// The address of this library's stream for work that runs beside the current stream (a
// hipStream_t as an integer, for torch.cuda.ExternalStream), or 0 when there is none (yet): it is
// created on the first call per device that is not under stream capture.
int64_t aux_stream(int64_t device) {
  c10::DeviceGuard guard(c10::Device(c10::DeviceType::CUDA, static_cast<c10::DeviceIndex>(device)));
  const hipStream_t current = c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(static_cast<c10::DeviceIndex>(device)).stream();
  SideStream* s = side_stream(static_cast<int>(device), current, 1);
  return s ? static_cast<int64_t>(reinterpret_cast<intptr_t>(s->stream)) : 0;
}

}  // namespace

TORCH_LIBRARY(mi355_moe, m) {
  m.def("aux_stream(int device) -> int", aux_stream);
  m.def("router_gate_fwd(Tensor x, Tensor w, Tensor? logit_bias) -> Tensor");
  m.def("router_gate_bwd(Tensor dlogits, Tensor x, Tensor w, bool need_dx, bool need_dw) -> (Tensor, Tensor)");
  m.def(
      "router_select_fwd(Tensor logits, Tensor? expert_bias, int top_k, int score_func, bool route_norm, "
      "float route_scale, int num_groups, int num_limited, int mode, bool want_scores, bool want_map) -> "
      "(Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "router_select_cutoff_fwd(Tensor logits, Tensor? expert_bias, int top_k, int score_func, bool route_norm, "
      "float route_scale) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "router_select_bwd(Tensor logits, Tensor ids, Tensor? dweights, Tensor? dscores, int score_func, "
      "bool route_norm, float route_scale, int mode) -> Tensor");
  m.def(
      "quantile_observe(Tensor(a!) histogram, Tensor scores, Tensor cutoff, Tensor expert_bias, "
      "Tensor? padding_mask) -> ()");
  m.def("quantile_estimate(Tensor histogram, Tensor expert_bias, int top_k) -> Tensor");
  m.def("rms_norm_fwd(Tensor x, Tensor weight, float epsilon) -> (Tensor, Tensor)");
  m.def(
      "rms_norm_bwd(Tensor dy, Tensor x, Tensor weight, Tensor rstd, bool need_dx, bool need_dw) -> (Tensor, Tensor)");
  m.def("balance_loss_fwd(Tensor scores, Tensor routing_map, Tensor? padding_mask) -> Tensor");
  m.def("balance_loss_bwd(Tensor scores, Tensor f, Tensor? padding_mask, Tensor grad_loss) -> Tensor");
  m.def(
      "permute_plan(Tensor ids, int num_experts, int local_lo, int local_hi, int align) -> (Tensor, Tensor, Tensor)");
  m.def("segments_from_counts(Tensor counts, int total_rows) -> Tensor");
  m.def(
      "permute_rows_fwd(Tensor x, Tensor row_of_slot, Tensor? slot_of_row, Tensor total_rows, int top_k, "
      "int row_capacity) -> Tensor");
  m.def("permute_rows_bwd(Tensor drows, Tensor row_of_slot, int num_tokens, int top_k) -> Tensor");
  m.def(
      "combine_fwd(Tensor y, Tensor weights, Tensor row_of_slot, Tensor? slot_of_row, Tensor? total_rows, "
      "int num_tokens, int top_k, bool round_terms) -> Tensor");
  m.def(
      "combine_bwd(Tensor dout, Tensor y, Tensor weights, Tensor row_of_slot, Tensor? slot_of_row, "
      "Tensor? total_rows, int top_k) -> (Tensor, Tensor)");
  m.def("combine_row_scale(Tensor weights, Tensor slot_of_row, int row_capacity) -> Tensor");
  m.def("combine_scores_bwd(Tensor dot_partial, Tensor row_of_slot, int num_tokens, int top_k) -> Tensor");
  m.def(
      "grouped_swiglu_fwd(Tensor rows, Tensor? token_of_row, Tensor w1, Tensor w3, Tensor w2, Tensor seg_offsets, "
      "Tensor seg_counts, Tensor tile_expert, Tensor tile_row0, Tensor num_tiles, int row_capacity, "
      "bool zero_fill) -> (Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "grouped_swiglu_bwd(Tensor dy, Tensor rows, Tensor? token_of_row, Tensor w1, Tensor w3, Tensor w2, "
      "Tensor gate, Tensor up, Tensor h, Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, "
      "Tensor tile_row0, Tensor num_tiles, bool need_drows, bool need_dw, bool zero_fill) -> "
      "(Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "grouped_linear_fwd(Tensor x, Tensor w, Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, "
      "Tensor tile_row0, Tensor num_tiles, bool zero_fill) -> Tensor");
  m.def(
      "grouped_linear_bwd(Tensor dy, Tensor x, Tensor w, Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, "
      "Tensor tile_row0, Tensor num_tiles, bool need_dx, bool need_dw, bool zero_fill) -> (Tensor, Tensor)");
  m.def(
      "rows_experts_combine_fwd(Tensor x, Tensor weights, Tensor w1, Tensor w3, Tensor w2, Tensor row_of_slot, "
      "Tensor? slot_of_row, Tensor total_rows, Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, "
      "Tensor tile_row0, Tensor num_tiles, int top_k, int row_capacity, bool round_terms) -> "
      "(Tensor, Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "rows_experts_combine_bwd(Tensor dout, Tensor rows, Tensor weights, Tensor w1, Tensor w3, Tensor w2, "
      "Tensor gate, Tensor up, Tensor h, Tensor y, Tensor row_of_slot, Tensor? slot_of_row, Tensor total_rows, "
      "Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, Tensor tile_row0, Tensor num_tiles, int num_tokens, "
      "int top_k, bool need_dx, bool need_dw) -> (Tensor, Tensor, Tensor, Tensor, Tensor)");
  m.def(
      "gather_experts_combine_fwd(Tensor x, Tensor weights, Tensor w1, Tensor w3, Tensor w2, Tensor token_of_row, "
      "Tensor slot_of_row, Tensor row_of_slot, Tensor seg_offsets, Tensor seg_counts, Tensor tile_expert, Tensor tile_row0, "
      "Tensor num_tiles, int top_k, int row_capacity, bool round_terms, bool save_gate_up) -> (Tensor, Tensor, Tensor)");
  m.def(
      "gather_experts_combine_bwd(Tensor dout, Tensor x, Tensor weights, Tensor w1, Tensor w3, Tensor w2, "
      "Tensor gate, Tensor up, Tensor token_of_row, Tensor slot_of_row, Tensor row_of_slot, Tensor seg_offsets, "
      "Tensor seg_counts, Tensor tile_expert, Tensor tile_row0, Tensor num_tiles, int top_k, bool need_dx, "
      "bool need_dw) -> (Tensor, Tensor, Tensor, Tensor, Tensor)");
}

TORCH_LIBRARY_IMPL(mi355_moe, CUDA, m) {
  m.impl("router_gate_fwd", router_gate_fwd);
  m.impl("router_gate_bwd", router_gate_bwd);
  m.impl("router_select_fwd", router_select_fwd);
  m.impl("router_select_cutoff_fwd", router_select_cutoff_fwd);
  m.impl("router_select_bwd", router_select_bwd);
  m.impl("quantile_observe", quantile_observe);
  m.impl("quantile_estimate", quantile_estimate);
  m.impl("rms_norm_fwd", rms_norm_fwd);
  m.impl("rms_norm_bwd", rms_norm_bwd);
  m.impl("balance_loss_fwd", balance_loss_fwd);
  m.impl("balance_loss_bwd", balance_loss_bwd);
  m.impl("permute_plan", permute_plan);
  m.impl("segments_from_counts", segments_from_counts);
  m.impl("permute_rows_fwd", permute_rows_fwd);
  m.impl("permute_rows_bwd", permute_rows_bwd);
  m.impl("combine_fwd", combine_fwd);
  m.impl("combine_bwd", combine_bwd);
  m.impl("combine_row_scale", combine_row_scale);
  m.impl("combine_scores_bwd", combine_scores_bwd);
  m.impl("grouped_swiglu_fwd", grouped_swiglu_fwd);
  m.impl("grouped_swiglu_bwd", grouped_swiglu_bwd);
  m.impl("grouped_linear_fwd", grouped_linear_fwd);
  m.impl("grouped_linear_bwd", grouped_linear_bwd);
  m.impl("rows_experts_combine_fwd", rows_experts_combine_fwd);
  m.impl("rows_experts_combine_bwd", rows_experts_combine_bwd);
  m.impl("gather_experts_combine_fwd", gather_experts_combine_fwd);
  m.impl("gather_experts_combine_bwd", gather_experts_combine_bwd);
}
