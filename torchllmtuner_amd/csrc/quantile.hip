// Quantile-balanced routing: the required-bias histogram and the bias estimate read from it
// (llmtuner/models/common/moe/routing.py:433-461 and :557-610).
//
// observe:   for every valid token t and expert e
//              required = cutoff[t] - scores[t][e]
//              bin      = clamp(floor((required - (min(bias) - 1)) / width), 0, B-1)
//              width    = (max(bias) - min(bias) + 2) / B
//              histogram[e][bin] += 1                        (int64 counters)
//            One thread per (t, e) pair, coalesced over the score map, 64-bit integer atomics:
//            integer adds commute, so the histogram does not depend on the order they land in.
//            The fp32 operations are the reference's, in its order, so that a pair falls into
//            the same bin.
// estimate:  per expert the K/E quantile of its histogram, interpolated inside the crossing
//            bin with the numerator kept integral, then mean-centred; one workgroup, one
//            wavefront per expert in turn (prefix sums by lane shuffles).
#include <algorithm>

#include "common.h"

namespace mi355 {
namespace {

// min and max of bias[0..E) in every thread of a 256-thread workgroup
__device__ __forceinline__ void bias_range(const float* __restrict__ bias, int E, float* red, float& mn,
                                           float& mx) {
  float lo = INFINITY, hi = -INFINITY;
  for (int e = threadIdx.x; e < E; e += 256) {
    lo = fminf(lo, bias[e]);
    hi = fmaxf(hi, bias[e]);
  }
  red[threadIdx.x] = lo;
  red[256 + threadIdx.x] = hi;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) {
      red[threadIdx.x] = fminf(red[threadIdx.x], red[threadIdx.x + o]);
      red[256 + threadIdx.x] = fmaxf(red[256 + threadIdx.x], red[256 + threadIdx.x + o]);
    }
    __syncthreads();
  }
  mn = red[0];
  mx = red[256];
}

__global__ __launch_bounds__(256) void quantile_observe_kernel(
    const float* __restrict__ scores, const float* __restrict__ cutoff, const float* __restrict__ bias,
    const uint8_t* __restrict__ padding, unsigned long long* __restrict__ hist, int T, int E, int B) {
#pragma clang fp contract(off)
  __shared__ float red[512];
  float mn, mx;
  bias_range(bias, E, red, mn, mx);
  const float lower = mn - 1.0f;
  const float width = ((mx - mn) + 2.0f) / static_cast<float>(B);
  const float top = static_cast<float>(B - 1);
  const int64_t total = static_cast<int64_t>(T) * E;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < total;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    const int t = static_cast<int>(i / E);
    const int e = static_cast<int>(i - static_cast<int64_t>(t) * E);
    if (padding && padding[t]) continue;
    const float required = cutoff[t] - scores[i];
    float q = floorf((required - lower) / width);
    q = fminf(fmaxf(q, 0.0f), top);  // also sends a NaN to bin 0 instead of out of range
    atomicAdd(hist + static_cast<int64_t>(e) * B + static_cast<int>(q), 1ull);
  }
}

// The same histogram through LDS: a workgroup owns `eg` neighbouring experts and a run of
// tokens, counts their pairs in 32-bit LDS bins (a call adds fewer than 2^31 pairs to a
// bin) and then adds its non-empty bins to the 64-bit histogram.  The required biases of
// one expert cluster in a few dozen bins, so this replaces most of the global atomics,
// which queue up on those few addresses, by LDS ones.
__global__ __launch_bounds__(256) void quantile_observe_lds_kernel(
    const float* __restrict__ scores, const float* __restrict__ cutoff, const float* __restrict__ bias,
    const uint8_t* __restrict__ padding, unsigned long long* __restrict__ hist, int T, int E, int B,
    int eg, int tokens_per_block) {
#pragma clang fp contract(off)
  extern __shared__ unsigned bins[];  // [eg][B]
  __shared__ float red[512];
  float mn, mx;
  bias_range(bias, E, red, mn, mx);
  const float lower = mn - 1.0f;
  const float width = ((mx - mn) + 2.0f) / static_cast<float>(B);
  const float top = static_cast<float>(B - 1);
  const int e0 = blockIdx.x * eg;
  const int ne = min(eg, E - e0);
  const int t0 = blockIdx.y * tokens_per_block;
  const int nt = min(tokens_per_block, T - t0);
  for (int i = threadIdx.x; i < eg * B; i += 256) bins[i] = 0u;
  __syncthreads();
  for (int i = threadIdx.x; i < nt * eg; i += 256) {
    const int t = t0 + i / eg, j = i % eg;
    if (j >= ne || (padding && padding[t])) continue;
    const float required = cutoff[t] - scores[static_cast<int64_t>(t) * E + e0 + j];
    float q = floorf((required - lower) / width);
    q = fminf(fmaxf(q, 0.0f), top);
    atomicAdd(bins + j * B + static_cast<int>(q), 1u);
  }
  __syncthreads();
  for (int i = threadIdx.x; i < ne * B; i += 256) {
    const unsigned c = bins[i];
    if (c) atomicAdd(hist + static_cast<int64_t>(e0) * B + i, static_cast<unsigned long long>(c));
  }
}

__device__ __forceinline__ long long wave_sum_i64(long long v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}

// Quantile position of every expert (in bins): one wavefront per expert.  pos_E[E] holds
// the positions, observed_E[e] whether expert e saw anything.
__global__ __launch_bounds__(256) void quantile_position_kernel(const long long* __restrict__ hist,
                                                                const float* __restrict__ bias,
                                                                float* __restrict__ pos, int* __restrict__ observed_E,
                                                                int E, int K, int B) {
#pragma clang fp contract(off)
  __shared__ float red[512];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float mn, mx;
  bias_range(bias, E, red, mn, mx);
  const float width = ((mx - mn) + 2.0f) / static_cast<float>(B);
  const float lower = mn - 1.0f;

  for (int e = blockIdx.x * 4 + wave; e < E; e += gridDim.x * 4) {
    const long long* row = hist + static_cast<int64_t>(e) * B;
    long long cnt = 0;
    for (int b = lane; b < B; b += 64) cnt += row[b];
    cnt = wave_sum_i64(cnt);
    const long long target_num = cnt * K;
    const long long target_rank = (target_num + E - 1) / E;
    // first bin whose inclusive prefix sum reaches the target rank
    long long running = 0, in_bin = 0, before = 0;
    int tbin = -1;
    for (int b0 = 0; b0 < B && tbin < 0; b0 += 64) {
      const int b = b0 + lane;
      const long long h = b < B ? row[b] : 0;
      long long incl = h;
#pragma unroll
      for (int o = 1; o < 64; o <<= 1) {
        const long long up = __shfl_up(incl, o, kWave);
        if (lane >= o) incl += up;
      }
      incl += running;
      const unsigned long long hit = __ballot(b < B && incl >= target_rank);
      if (hit) {
        const int l = __ffsll(static_cast<long long>(hit)) - 1;
        tbin = b0 + l;
        in_bin = __shfl(h, l, kWave);
        before = __shfl(incl, l, kWave) - in_bin;
      }
      running = __shfl(incl, 63, kWave);
    }
    if (tbin < 0) {  // only with negative counters: stay inside the histogram
      tbin = B - 1;
      in_bin = row[B - 1];
      before = running - in_bin;
    }
    if (lane == 0) {
      const float safe = fmaxf(static_cast<float>(in_bin), 1.0f);
      const long long residual = target_num - before * E;
      const float fraction = static_cast<float>(residual) / static_cast<float>(E) / safe;
      float p = static_cast<float>(tbin) + fraction;
      // an expert that saw nothing keeps its place
      if (cnt == 0) p = (bias[e] - lower) / width;
      pos[e] = p;
      observed_E[e] = cnt != 0;
    }
  }
}

// Mean-centring of the positions, in one workgroup and a fixed summation order.
__global__ __launch_bounds__(256) void quantile_centre_kernel(const float* __restrict__ pos,
                                                              const int* __restrict__ observed_E,
                                                              const float* __restrict__ bias,
                                                              float* __restrict__ out, int E, int B) {
#pragma clang fp contract(off)
  __shared__ float red[512];
  __shared__ int observed;  // some expert has a non-empty histogram
  if (threadIdx.x == 0) observed = 0;
  float mn, mx;
  bias_range(bias, E, red, mn, mx);  // its barriers also publish `observed = 0`
  const float width = ((mx - mn) + 2.0f) / static_cast<float>(B);
  int any = 0;
  for (int e = threadIdx.x; e < E; e += 256) any |= observed_E[e];
  if (any) observed = 1;
  __syncthreads();
  if (!observed) {  // no valid token at all: the bias comes back bit for bit
    for (int e = threadIdx.x; e < E; e += 256) out[e] = bias[e];
    return;
  }
  float part = 0.0f;
  for (int e = threadIdx.x; e < E; e += 256) part += pos[e];
  red[threadIdx.x] = part;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if (threadIdx.x < o) red[threadIdx.x] += red[threadIdx.x + o];
    __syncthreads();
  }
  const float mean = red[0] / static_cast<float>(E);
  for (int e = threadIdx.x; e < E; e += 256) out[e] = (pos[e] - mean) * width;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_quantile_observe(const float* scores_TE, const float* cutoff_T,
                                      const float* expert_bias_E, const uint8_t* padding_mask_T,
                                      int64_t* histogram_EB, int64_t T, int64_t E, int64_t B,
                                      void* stream) {
  MI355_REQUIRE(T >= 0 && T < (1ll << 31) && E >= 1 && E <= (1 << 20) && B >= 1 && B < (1 << 24),
                "quantile_observe: bad shape T=%lld E=%lld B=%lld", (long long)T, (long long)E, (long long)B);
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(scores_TE && cutoff_T && expert_bias_E && histogram_EB, "quantile_observe: null pointer");
  unsigned long long* hist = reinterpret_cast<unsigned long long*>(histogram_EB);
  // experts per workgroup: what 32 KiB of LDS bins hold, at most 4 (more workgroups)
  const int64_t eg = std::min<int64_t>(std::min<int64_t>(4, E), (32 * 1024) / (B * 4));
  if (eg >= 1 && T >= 256) {
    const int64_t groups = (E + eg - 1) / eg;
    // about 256 workgroups, each with at least 256 tokens so that the LDS bins pay off
    const int64_t chunks = std::max<int64_t>(1, std::min<int64_t>(T / 256, (256 + groups - 1) / groups));
    const int64_t per = (T + chunks - 1) / chunks;
    hipLaunchKernelGGL(quantile_observe_lds_kernel, dim3((unsigned)groups, (unsigned)((T + per - 1) / per)),
                       dim3(256), (size_t)(eg * B * 4), as_stream(stream), scores_TE, cutoff_T, expert_bias_E,
                       padding_mask_T, hist, (int)T, (int)E, (int)B, (int)eg, (int)per);
    return check_launch("quantile_observe");
  }
  const int64_t total = T * E;
  const unsigned blocks = (unsigned)std::min<int64_t>((total + 255) / 256, 4096);
  hipLaunchKernelGGL(quantile_observe_kernel, dim3(blocks), dim3(256), 0, as_stream(stream), scores_TE,
                     cutoff_T, expert_bias_E, padding_mask_T, hist, (int)T, (int)E, (int)B);
  return check_launch("quantile_observe");
}

extern "C" int mi355_quantile_estimate(const int64_t* histogram_EB, const float* expert_bias_E,
                                       float* next_bias_E, void* workspace, int64_t E, int64_t K,
                                       int64_t B, void* stream) {
  MI355_REQUIRE(E >= 1 && E <= 8192 && B >= 1 && B < (1 << 24) && K >= 1 && K < E,
                "quantile_estimate: bad shape E=%lld K=%lld B=%lld (0 < K < E <= 8192)", (long long)E,
                (long long)K, (long long)B);
  MI355_REQUIRE(histogram_EB && expert_bias_E && next_bias_E && workspace, "quantile_estimate: null pointer");
  float* pos = static_cast<float*>(workspace);
  int* observed = reinterpret_cast<int*>(pos + E);
  hipLaunchKernelGGL(quantile_position_kernel, dim3((unsigned)((E + 3) / 4)), dim3(256), 0, as_stream(stream),
                     reinterpret_cast<const long long*>(histogram_EB), expert_bias_E, pos, observed, (int)E,
                     (int)K, (int)B);
  hipLaunchKernelGGL(quantile_centre_kernel, dim3(1), dim3(256), 0, as_stream(stream), pos, observed,
                     expert_bias_E, next_bias_E, (int)E, (int)B);
  return check_launch("quantile_estimate");
}
