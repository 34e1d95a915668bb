// Per-forward load-balance loss of the router (DeepSeek-V3 eqs. 17-19 in the T-free form
// the reference uses) and its gradient with respect to the dense score map.
//
//   counts_e = sum_t map[t][e]             f_e = E * counts_e / max(sum_e counts_e, 1e-12)
//   s'_{t,e} = s_{t,e} / max(sum_e s_{t,e}, 1e-12), zero for padding tokens
//   p_e      = sum_t s'_{t,e}              loss = sum_e f_e * p_e
//
// The routing map is piecewise constant, so the gradient reaches the scores through p
// only:  d loss / d s_{t,j} = (f_j - sum_e f_e s'_{t,e}) / S_t.
// One wavefront per token, lane l holds experts l, l+64, ...; per-workgroup partial sums
// are combined in a fixed order, so the result is deterministic.
#include "common.h"

namespace mi355 {
namespace {

constexpr int kTokPerBlock = 64;   // tokens per workgroup of 4 waves
constexpr int kMaxVpl = 16;        // experts per lane: E <= 1024
constexpr float kEps = 1e-12f;     // F.normalize's clamp

__global__ __launch_bounds__(256) void balance_partial_kernel(
    const float* __restrict__ scores, const uint8_t* __restrict__ map,
    const uint8_t* __restrict__ padding, float* __restrict__ partial, int T, int E) {
  extern __shared__ float lds[];  // [4 waves][2][E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float p[kMaxVpl], c[kMaxVpl];
#pragma unroll
  for (int j = 0; j < kMaxVpl; ++j) p[j] = c[j] = 0.0f;
  const int t0 = blockIdx.x * kTokPerBlock;
  for (int i = wave; i < kTokPerBlock; i += 4) {
    const int t = t0 + i;
    if (t >= T) break;  // uniform per wave
    const float* row = scores + static_cast<int64_t>(t) * E;
    const uint8_t* mrow = map + static_cast<int64_t>(t) * E;
    float s[kMaxVpl];
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxVpl; ++j) {
      const int e = lane + 64 * j;
      s[j] = e < E ? row[e] : 0.0f;
      sum += s[j];
      if (e < E) c[j] += mrow[e] ? 1.0f : 0.0f;
    }
    sum = wave_sum(sum);
    const bool pad = padding && padding[t];
    const float inv = pad ? 0.0f : 1.0f / fmaxf(sum, kEps);
#pragma unroll
    for (int j = 0; j < kMaxVpl; ++j) p[j] += s[j] * inv;
  }
  float* mine = lds + wave * 2 * E;
#pragma unroll
  for (int j = 0; j < kMaxVpl; ++j) {
    const int e = lane + 64 * j;
    if (e < E) { mine[e] = p[j]; mine[E + e] = c[j]; }
  }
  __syncthreads();
  for (int e = threadIdx.x; e < 2 * E; e += 256) {
    const float v = ((lds[e] + lds[2 * E + e]) + lds[4 * E + e]) + lds[6 * E + e];
    partial[static_cast<int64_t>(blockIdx.x) * 2 * E + e] = v;
  }
}

__global__ __launch_bounds__(256) void balance_final_kernel(const float* __restrict__ partial, int nblk,
                                                            float* __restrict__ f_E, float* __restrict__ loss,
                                                            int E) {
  extern __shared__ float lds[];  // p[E], c[E], red[256]
  float* p = lds;
  float* c = lds + E;
  float* red = lds + 2 * E;
  for (int e = threadIdx.x; e < 2 * E; e += 256) {
    float acc = 0.0f;
    for (int b = 0; b < nblk; ++b) acc += partial[static_cast<int64_t>(b) * 2 * E + e];
    lds[e] = acc;
  }
  __syncthreads();
  float part = 0.0f;
  for (int e = threadIdx.x; e < E; e += 256) part += c[e];
  red[threadIdx.x] = part;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  const float scale = static_cast<float>(E) / fmaxf(red[0], kEps);
  __syncthreads();
  part = 0.0f;
  for (int e = threadIdx.x; e < E; e += 256) {
    const float f = c[e] * scale;
    f_E[e] = f;
    part += f * p[e];
  }
  red[threadIdx.x] = part;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) loss[0] = red[0];
}

__global__ __launch_bounds__(256) void balance_bwd_kernel(
    const float* __restrict__ scores, const float* __restrict__ f_E, const uint8_t* __restrict__ padding,
    const float* __restrict__ gloss, float* __restrict__ dscores, int T, int E) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;
  const float g = gloss[0];
  const float* row = scores + static_cast<int64_t>(t) * E;
  float* out = dscores + static_cast<int64_t>(t) * E;
  float s[kMaxVpl], f[kMaxVpl];
  float sum = 0.0f, dot = 0.0f;
#pragma unroll
  for (int j = 0; j < kMaxVpl; ++j) {
    const int e = lane + 64 * j;
    s[j] = e < E ? row[e] : 0.0f;
    f[j] = e < E ? f_E[e] : 0.0f;
    sum += s[j];
    dot += s[j] * f[j];
  }
  sum = wave_sum(sum);
  dot = wave_sum(dot);
  const bool pad = padding && padding[t];
  // below the clamp the normalised score is s / eps and the sum no longer enters
  const bool clamped = sum < kEps;
  const float inv = 1.0f / fmaxf(sum, kEps);
  const float mean = clamped ? 0.0f : dot * inv;
#pragma unroll
  for (int j = 0; j < kMaxVpl; ++j) {
    const int e = lane + 64 * j;
    if (e < E) out[e] = pad ? 0.0f : g * (f[j] - mean) * inv;
  }
}

int nblk_for(int64_t T) { return static_cast<int>((T + kTokPerBlock - 1) / kTokPerBlock); }

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int64_t mi355_balance_loss_workspace_bytes(int64_t T, int64_t E) {
  if (T < 0 || E < 1) return 0;
  return static_cast<int64_t>(nblk_for(T)) * 2 * E * 4;
}

extern "C" int mi355_balance_loss_fwd(const float* scores_TE, const uint8_t* routing_map_TE,
                                      const uint8_t* padding_mask_T, float* loss, float* f_E,
                                      void* workspace, int64_t T, int64_t E, void* stream) {
  MI355_REQUIRE(T >= 0 && E >= 1 && E <= 64 * kMaxVpl && T < (1ll << 31),
                "balance_loss_fwd: bad shape T=%lld E=%lld (E <= 1024)", (long long)T, (long long)E);
  MI355_REQUIRE(loss && f_E, "balance_loss_fwd: null output");
  MI355_REQUIRE(T == 0 || (scores_TE && routing_map_TE && workspace), "balance_loss_fwd: null pointer");
  hipStream_t s = as_stream(stream);
  const int nblk = nblk_for(T);
  if (nblk > 0)
    hipLaunchKernelGGL(balance_partial_kernel, dim3(nblk), dim3(256), (size_t)8 * E * sizeof(float), s, scores_TE,
                       routing_map_TE, padding_mask_T, static_cast<float*>(workspace), (int)T, (int)E);
  hipLaunchKernelGGL(balance_final_kernel, dim3(1), dim3(256), (size_t)(2 * E + 256) * sizeof(float), s,
                     static_cast<const float*>(workspace), nblk, f_E, loss, (int)E);
  return check_launch("balance_loss_fwd");
}

extern "C" int mi355_balance_loss_bwd(const float* scores_TE, const float* f_E,
                                      const uint8_t* padding_mask_T, const float* grad_loss,
                                      float* dscores_TE, int64_t T, int64_t E, void* stream) {
  MI355_REQUIRE(T >= 0 && E >= 1 && E <= 64 * kMaxVpl && T < (1ll << 31), "balance_loss_bwd: bad shape");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(scores_TE && f_E && grad_loss && dscores_TE, "balance_loss_bwd: null pointer");
  hipLaunchKernelGGL(balance_bwd_kernel, dim3((unsigned)((T + 3) / 4)), dim3(256), 0, as_stream(stream), scores_TE,
                     f_E, padding_mask_T, grad_loss, dscores_TE, (int)T, (int)E);
  return check_launch("balance_loss_bwd");
}
