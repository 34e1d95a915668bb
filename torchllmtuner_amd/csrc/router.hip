// Router: fp32 gate projection and the fused score / top-k / gather / norm pass.
//
// Selection kernels: a token is owned by one row of 16 lanes (E = 64, 128 or 256: four tokens
// per wavefront, lane l keeps experts l*E/16 ...) or by one 64-lane wavefront (any E up to 512:
// lane l keeps experts l, l+64, l+128, ...).  The scores stay in registers, the softmax max /
// sum and every arg-max are DPP reductions, and the K winners are written by lanes 0..K-1.  No
// LDS, no atomics; HBM traffic is the (T,E) logits once plus the (T,K) outputs.
#include <type_traits>

#include "common.h"
#include "gemm_generic.h"

namespace mi355 {
namespace {

constexpr int kMaxVPL = 8;  // experts per lane -> E <= 512
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float softplus_f32(float x) {
  return x > 20.0f ? x : log1pf(expf(x));  // torch's threshold=20, beta=1
}

// Wave reductions of this file run on DPP row operations (VALU rate) plus four lane reads, not on
// shuffles: a shuffle is an LDS permute, and a token's selection needs about a hundred of them --
// with one wavefront per token the LDS pipe of a CU, not memory, was what the select kernels waited
// for.  The four controls below exchange within a row of 16 lanes (pairs, quads, halves, the row),
// so after them every lane holds its row's result; lanes 0, 16, 32, 48 then give the four rows.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false);
}
constexpr int kDppPairs = 0xB1, kDppQuads = 0x4E, kDppHalfMirror = 0x141, kDppRowMirror = 0x140;

__device__ __forceinline__ float lane_f32(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}

// sum over the wave, left in every lane
__device__ __forceinline__ float wave_sum_dpp(float v) {
  v += dpp_f32<kDppPairs>(v);
  v += dpp_f32<kDppQuads>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  v += dpp_f32<kDppRowMirror>(v);
  return (lane_f32(v, 0) + lane_f32(v, 16)) + (lane_f32(v, 32) + lane_f32(v, 48));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
  v = fmaxf(v, dpp_f32<kDppPairs>(v));
  v = fmaxf(v, dpp_f32<kDppQuads>(v));
  v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
  v = fmaxf(v, dpp_f32<kDppRowMirror>(v));
  return fmaxf(fmaxf(lane_f32(v, 0), lane_f32(v, 16)), fmaxf(lane_f32(v, 32), lane_f32(v, 48)));
}

// the better of two (value, index) candidates: the larger value, ties to the lower index
__device__ __forceinline__ void take_better(float& v, int& idx, float ov, int oi) {
  if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; }
}

// (value, index) arg-max across the wave, left in every lane; ties go to the lower index.
__device__ __forceinline__ void wave_argmax(float& v, int& idx) {
  { const float ov = dpp_f32<kDppPairs>(v); const int oi = dpp_i32<kDppPairs>(idx); take_better(v, idx, ov, oi); }
  { const float ov = dpp_f32<kDppQuads>(v); const int oi = dpp_i32<kDppQuads>(idx); take_better(v, idx, ov, oi); }
  { const float ov = dpp_f32<kDppHalfMirror>(v); const int oi = dpp_i32<kDppHalfMirror>(idx); take_better(v, idx, ov, oi); }
  { const float ov = dpp_f32<kDppRowMirror>(v); const int oi = dpp_i32<kDppRowMirror>(idx); take_better(v, idx, ov, oi); }
  float a = lane_f32(v, 0), b = lane_f32(v, 32);
  int ai = __builtin_amdgcn_readlane(idx, 0), bi = __builtin_amdgcn_readlane(idx, 32);
  take_better(a, ai, lane_f32(v, 16), __builtin_amdgcn_readlane(idx, 16));
  take_better(b, bi, lane_f32(v, 48), __builtin_amdgcn_readlane(idx, 48));
  take_better(a, ai, b, bi);
  v = a;
  idx = ai;
}

// the two largest of {a1 >= a2} and {b1 >= b2}, equal values counted as often as they occur
__device__ __forceinline__ void merge_top2(float& a1, float& a2, float b1, float b2) {
  const float lo = fminf(a1, b1);
  a1 = fmaxf(a1, b1);
  a2 = fmaxf(lo, fmaxf(a2, b2));
}
template <int CTRL>
__device__ __forceinline__ void top2_dpp(float& m1, float& m2) {
  const float o1 = dpp_f32<CTRL>(m1), o2 = dpp_f32<CTRL>(m2);
  merge_top2(m1, m2, o1, o2);
}
// The two largest values held by the `width` lanes (a power of two, 2..64; wave-uniform) of every
// aligned run of lanes, left in all of them.  Each step exchanges between two halves that already
// agree among themselves, so the mirrors of the DPP controls are as good as a butterfly.
__device__ __forceinline__ void run_top2(float& m1, float& m2, int width) {
  top2_dpp<kDppPairs>(m1, m2);
  if (width >= 4) top2_dpp<kDppQuads>(m1, m2);
  if (width >= 8) top2_dpp<kDppHalfMirror>(m1, m2);
  if (width >= 16) top2_dpp<kDppRowMirror>(m1, m2);
  if (width >= 32) {
    // lane ^ 16 within each half of the wave (swizzle bit mode: and 0x1f, or 0, xor 0x10)
    const float o1 = __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(m1), 0x401f));
    const float o2 = __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(m2), 0x401f));
    merge_top2(m1, m2, o1, o2);
  }
  if (width >= 64) {
    float a1 = lane_f32(m1, 0), a2 = lane_f32(m2, 0);
    merge_top2(a1, a2, lane_f32(m1, 32), lane_f32(m2, 32));
    m1 = a1;
    m2 = a2;
  }
}

template <int VPL>
__device__ __forceinline__ float pick(const float (&a)[VPL], int j) {
  float r = a[0];
#pragma unroll
  for (int q = 1; q < VPL; ++q) r = (j == q) ? a[q] : r;
  return r;
}

template <int VPL>
__device__ __forceinline__ void compute_scores(const float* __restrict__ row, int E, int lane,
                                               int score_func, float (&s)[VPL], float (&x)[VPL]) {
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + j * kWave;
    x[j] = e < E ? row[e] : -INFINITY;
  }
  if (score_func == MI355_SCORE_SOFTMAX) {
    float m = x[0];
#pragma unroll
    for (int j = 1; j < VPL; ++j) m = fmaxf(m, x[j]);
    m = wave_max_dpp(m);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      s[j] = (lane + j * kWave < E) ? expf(x[j] - m) : 0.0f;
      sum += s[j];
    }
    sum = wave_sum_dpp(sum);
#pragma unroll
    for (int j = 0; j < VPL; ++j) s[j] = s[j] / sum;
  } else if (score_func == MI355_SCORE_SIGMOID) {
#pragma unroll
    for (int j = 0; j < VPL; ++j) s[j] = 1.0f / (1.0f + expf(-x[j]));
  } else {
#pragma unroll
    for (int j = 0; j < VPL; ++j) s[j] = sqrtf(softplus_f32(x[j]));
  }
}

template <int VPL>
__global__ __launch_bounds__(256) void select_fwd_kernel(
    const float* __restrict__ logits, const float* __restrict__ expert_bias,
    float* __restrict__ weights, int64_t* __restrict__ ids, float* __restrict__ scores_out,
    uint8_t* __restrict__ map_out, float* __restrict__ cutoff_out, int T, int E, int K, int score_func,
    int route_norm,
    float route_scale, int num_groups, int num_limited, int mode) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T) return;

  float s[VPL], x[VPL];
  compute_scores<VPL>(logits + static_cast<int64_t>(t) * E, E, lane, score_func, s, x);
  if (scores_out) {
#pragma unroll
    for (int j = 0; j < VPL; ++j)
      if (lane + j * kWave < E) scores_out[static_cast<int64_t>(t) * E + lane + j * kWave] = s[j];
  }

  float my_w = 0.0f;
  int my_id = 0;

  if (mode == MI355_SELECT_TOPK) {
    // Choice values.  Without a bias and without groups the choice is the plain top-k of the
    // scores, and every score function here is non-decreasing in the logit: the experts are
    // then chosen by LOGIT, which is exact -- two implementations of exp() that differ in the
    // last ulp can order two nearly equal scores differently, but never two logits.
    // (not when the caller asks for the cutoff: that is a choice VALUE, the (K+1)-th score)
    const bool by_logit = !expert_bias && num_groups == 0 && !cutoff_out;
    float c[VPL];
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = lane + j * kWave;
      c[j] = e < E ? (by_logit ? x[j] : (expert_bias ? s[j] + expert_bias[e] : s[j])) : -INFINITY;
    }
    unsigned taken = 0;
#pragma unroll
    for (int j = 0; j < VPL; ++j)
      if (lane + j * kWave >= E) taken |= 1u << j;  // never selectable

    if (num_groups > 0) {
      // group score = sum of the group's two best choice scores; keep the best
      // num_limited groups (ties to the lower group), mask the rest to -inf.
      const int P = E / num_groups;
      float gscore = -INFINITY;  // lane g (< num_groups) keeps group g's score
      if (P < kWave && kWave % P == 0) {
        // a group is an aligned run of P lanes of one register: the registers' runs are reduced side
        // by side (independent chains), then lane g fetches the sum of its group's run
        const int runs = kWave / P;  // groups per register
        float sum[VPL];
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          float m1 = c[j], m2 = -INFINITY;
          run_top2(m1, m2, P);
          sum[j] = m1 + m2;
        }
        const int from = (lane % runs) * P;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          const float got = __int_as_float(__builtin_amdgcn_ds_bpermute(from << 2, __float_as_int(sum[j])));
          if (lane / runs == j) gscore = got;
        }
      } else if (P % kWave == 0) {
        // a group is P / 64 whole registers: each lane folds its own values, then one wave-wide step
        const int regs = P / kWave;
        float m1 = -INFINITY, m2 = -INFINITY;
#pragma unroll
        for (int j = 0; j < VPL; ++j) {
          merge_top2(m1, m2, c[j], -INFINITY);
          if ((j + 1) % regs == 0) {
            run_top2(m1, m2, kWave);
            if (lane == j / regs) gscore = m1 + m2;
            m1 = m2 = -INFINITY;
          }
        }
      } else {
        for (int g = 0; g < num_groups; ++g) {
          float top2 = 0.0f;
          unsigned used = 0;
          for (int r = 0; r < 2; ++r) {
            float bv = -INFINITY;
            int bi = 0x7fffffff;
#pragma unroll
            for (int j = 0; j < VPL; ++j) {
              const int e = lane + j * kWave;
              const bool in = e < E && e / P == g && !((used >> j) & 1u);
              if (in && (c[j] > bv || bi == 0x7fffffff)) { bv = c[j]; bi = e; }
            }
            wave_argmax(bv, bi);
            top2 += bv;
            if ((bi & 63) == lane) used |= 1u << (bi >> 6);
          }
          if (lane == g) gscore = top2;
        }
      }
      // a group is kept when fewer than num_limited groups beat it (a higher score, or the same
      // score and a lower index): the groups a repeated arg-max would pick, without the repeats
      const float mine = lane < num_groups ? gscore : -INFINITY;
      int beaten_by = 0;
      for (int g = 0; g < num_groups; ++g) {
        const float sg = lane_f32(gscore, g);
        beaten_by += (sg > mine || (sg == mine && g < lane)) ? 1 : 0;
      }
      const unsigned long long keep = __ballot(lane < num_groups && beaten_by < num_limited);
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        const int e = lane + j * kWave;
        if (e < E && !((keep >> (e / P)) & 1ull)) c[j] = -INFINITY;
      }
    }

    for (int k = 0; k < K; ++k) {
      float bv = -INFINITY;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        if ((taken >> j) & 1u) continue;
        if (bi == 0x7fffffff || c[j] > bv) { bv = c[j]; bi = lane + j * kWave; }
      }
      wave_argmax(bv, bi);
      const int owner = __builtin_amdgcn_readfirstlane(bi & 63), slot = bi >> 6;
      float sv = 0.0f;
      if (lane == owner) {
        taken |= 1u << slot;
        sv = pick<VPL>(s, slot);
      }
      sv = lane_f32(sv, owner);  // owner is wave-uniform: a lane read, not a shuffle
      if (lane == k) { my_w = sv; my_id = bi; }
    }
    if (cutoff_out) {
      // the best choice score left after the K winners: the (K+1)-th of a sorted top-(K+1)
      float bv = -INFINITY;
      int bi = 0x7fffffff;
#pragma unroll
      for (int j = 0; j < VPL; ++j) {
        if ((taken >> j) & 1u) continue;
        if (bi == 0x7fffffff || c[j] > bv) { bv = c[j]; bi = lane + j * kWave; }
      }
      wave_argmax(bv, bi);
      if (lane == 0) cutoff_out[t] = bv;
    }
  } else {
    // fixed: (t + k) % E ; balanced: (t*K + k) % E ; lane k owns slot k (K <= 64)
    const int64_t base = mode == MI355_SELECT_FIXED ? static_cast<int64_t>(t) + lane
                                                    : static_cast<int64_t>(t) * K + lane;
    my_id = static_cast<int>(base % E);
    // gather the unbiased score of each slot's expert from its owner lane
    for (int k = 0; k < K; ++k) {
      const int want = __builtin_amdgcn_readlane(my_id, k);
      const float got = lane_f32(pick<VPL>(s, want >> 6), __builtin_amdgcn_readfirstlane(want & 63));
      if (lane == k) my_w = got;
    }
  }

  if (mode == MI355_SELECT_FIXED) {
    my_w = 1.0f / static_cast<float>(K);
  } else {
    if (route_norm) {
      const float sum = wave_sum_dpp(lane < K ? my_w : 0.0f);
      my_w = my_w / (sum + 1e-20f);
    }
    my_w = my_w * route_scale;
  }
  if (lane < K) {
    weights[static_cast<int64_t>(t) * K + lane] = my_w;
    ids[static_cast<int64_t>(t) * K + lane] = my_id;
  }
  if (map_out) {
    // one-hot routing map of the token, one byte per expert
    unsigned chosen = 0;
    for (int k = 0; k < K; ++k) {
      const int idk = __builtin_amdgcn_readlane(my_id, k);
      if ((idk & 63) == lane) chosen |= 1u << (idk >> 6);
    }
#pragma unroll
    for (int j = 0; j < VPL; ++j)
      if (lane + j * kWave < E) map_out[static_cast<int64_t>(t) * E + lane + j * kWave] = (chosen >> j) & 1u;
  }
}

// ---- the same selection with one token per row of 16 lanes -------------------------------------
// For E = 64, 128 or 256, K <= 16 and 1, 2, 4, 8 or 16 expert groups (or none): four tokens per
// wavefront, lane l of a row keeps experts l*VPR .. l*VPR + VPR - 1, so a group is a run of
// 16 / num_groups whole lanes.  Every reduction is four
// DPP steps inside the row and serves four tokens at once, where the wave-per-token kernel above
// spends the same steps plus eight lane reads on one: the selection is bound by instruction
// issue, not by memory, and this form issues about a third of the instructions per token.  The
// choice (larger value, ties to the lower expert index) does not depend on the order of the
// comparisons, so both kernels pick the same experts.
__device__ __forceinline__ float row_max(float v) {
  v = fmaxf(v, dpp_f32<kDppPairs>(v));
  v = fmaxf(v, dpp_f32<kDppQuads>(v));
  v = fmaxf(v, dpp_f32<kDppHalfMirror>(v));
  return fmaxf(v, dpp_f32<kDppRowMirror>(v));
}
__device__ __forceinline__ float row_sum(float v) {
  v += dpp_f32<kDppPairs>(v);
  v += dpp_f32<kDppQuads>(v);
  v += dpp_f32<kDppHalfMirror>(v);
  return v + dpp_f32<kDppRowMirror>(v);
}
template <int CTRL>
__device__ __forceinline__ void row_better(float& v, int& idx, float& carried) {
  const float ov = dpp_f32<CTRL>(v), oc = dpp_f32<CTRL>(carried);
  const int oi = dpp_i32<CTRL>(idx);
  if (ov > v || (ov == v && oi < idx)) { v = ov; idx = oi; carried = oc; }
}
// (value, index) arg-max over a row, with a value carried along from the winner; left in all 16 lanes
__device__ __forceinline__ void row_argmax(float& v, int& idx, float& carried) {
  row_better<kDppPairs>(v, idx, carried);
  row_better<kDppQuads>(v, idx, carried);
  row_better<kDppHalfMirror>(v, idx, carried);
  row_better<kDppRowMirror>(v, idx, carried);
}

template <int VPR>
__global__ __launch_bounds__(256) void select_rows_kernel(
    const float* __restrict__ logits, const float* __restrict__ expert_bias, float* __restrict__ weights,
    int64_t* __restrict__ ids, float* __restrict__ scores_out, uint8_t* __restrict__ map_out,
    float* __restrict__ cutoff_out, int T, int K, int score_func, int route_norm, float route_scale,
    int num_groups, int num_limited) {
  constexpr int E = 16 * VPR;
  const int l = threadIdx.x & 15;
  const int t_raw = blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool live = t_raw < T;
  const int t = live ? t_raw : T - 1;  // a row past the end redoes the last token and stores nothing
  const int e0 = l * VPR;

  float x[VPR], s[VPR];
  const f32x4* src = reinterpret_cast<const f32x4*>(logits + static_cast<int64_t>(t) * E + e0);
#pragma unroll
  for (int q = 0; q < VPR / 4; ++q) {
    const f32x4 v = src[q];
    x[q * 4] = v[0]; x[q * 4 + 1] = v[1]; x[q * 4 + 2] = v[2]; x[q * 4 + 3] = v[3];
  }
  if (score_func == MI355_SCORE_SOFTMAX) {
    float m = x[0];
#pragma unroll
    for (int j = 1; j < VPR; ++j) m = fmaxf(m, x[j]);
    m = row_max(m);
    float sum = 0.0f;
#pragma unroll
    for (int j = 0; j < VPR; ++j) {
      s[j] = expf(x[j] - m);
      sum += s[j];
    }
    sum = row_sum(sum);
#pragma unroll
    for (int j = 0; j < VPR; ++j) s[j] = s[j] / sum;
  } else if (score_func == MI355_SCORE_SIGMOID) {
#pragma unroll
    for (int j = 0; j < VPR; ++j) s[j] = 1.0f / (1.0f + expf(-x[j]));
  } else {
#pragma unroll
    for (int j = 0; j < VPR; ++j) s[j] = sqrtf(softplus_f32(x[j]));
  }
  if (scores_out && live) {
    f32x4* dst = reinterpret_cast<f32x4*>(scores_out + static_cast<int64_t>(t) * E + e0);
#pragma unroll
    for (int q = 0; q < VPR / 4; ++q) {
      const f32x4 v = {s[q * 4], s[q * 4 + 1], s[q * 4 + 2], s[q * 4 + 3]};
      dst[q] = v;
    }
  }

  // choice values: the logit itself when nothing but a monotone score function stands between
  // it and the choice (exact: two exp() implementations can order two nearly equal scores
  // differently, never two logits), else score (+ bias)
  float c[VPR];
  if (expert_bias) {
    const f32x4* bsrc = reinterpret_cast<const f32x4*>(expert_bias + e0);
#pragma unroll
    for (int q = 0; q < VPR / 4; ++q) {
      const f32x4 b = bsrc[q];
#pragma unroll
      for (int i = 0; i < 4; ++i) c[q * 4 + i] = s[q * 4 + i] + b[i];
    }
  } else {
#pragma unroll
    for (int j = 0; j < VPR; ++j) c[j] = (num_groups > 0 || cutoff_out) ? s[j] : x[j];  // the cutoff is a score
  }
  if (num_groups > 0) {
    // group score = sum of the group's two best choice values: each lane folds its own, the lanes
    // of a group join them; every lane then counts the groups that beat its own (a higher score,
    // or the same score and a lower index), seeing each other group's score by a row rotation,
    // and a group beaten by num_limited others or more is masked
    const int m = 16 / num_groups;  // lanes per group
    float m1 = -INFINITY, m2 = -INFINITY;
#pragma unroll
    for (int j = 0; j < VPR; ++j) merge_top2(m1, m2, c[j], -INFINITY);
    if (m >= 2) top2_dpp<kDppPairs>(m1, m2);
    if (m >= 4) top2_dpp<kDppQuads>(m1, m2);
    if (m >= 8) top2_dpp<kDppHalfMirror>(m1, m2);
    if (m >= 16) top2_dpp<kDppRowMirror>(m1, m2);
    const float gs = m1 + m2;
    const int gid = l / m;
    int beaten_by = 0;
    auto other = [&](auto n_t) {
      constexpr int n = decltype(n_t)::value;
      if (n % m != 0) return;  // wave-uniform
      const float og = dpp_f32<0x120 + n>(gs);  // row rotation by n lanes
      const int oi = dpp_i32<0x120 + n>(gid);
      beaten_by += (og > gs || (og == gs && oi < gid)) ? 1 : 0;
    };
    other(std::integral_constant<int, 1>{}); other(std::integral_constant<int, 2>{});
    other(std::integral_constant<int, 3>{}); other(std::integral_constant<int, 4>{});
    other(std::integral_constant<int, 5>{}); other(std::integral_constant<int, 6>{});
    other(std::integral_constant<int, 7>{}); other(std::integral_constant<int, 8>{});
    other(std::integral_constant<int, 9>{}); other(std::integral_constant<int, 10>{});
    other(std::integral_constant<int, 11>{}); other(std::integral_constant<int, 12>{});
    other(std::integral_constant<int, 13>{}); other(std::integral_constant<int, 14>{});
    other(std::integral_constant<int, 15>{});
    if (beaten_by >= num_limited) {
#pragma unroll
      for (int j = 0; j < VPR; ++j) c[j] = -INFINITY;
    }
  }

  unsigned taken = 0;
  float my_w = 0.0f;
  int my_id = 0;
  auto best_left = [&](float& bv, int& bi, float& bs) {
    bv = -INFINITY;
    bi = 0x7fffffff;
    bs = 0.0f;
#pragma unroll
    for (int j = 0; j < VPR; ++j) {
      if ((taken >> j) & 1u) continue;
      if (bi == 0x7fffffff || c[j] > bv) { bv = c[j]; bi = e0 + j; bs = s[j]; }
    }
    row_argmax(bv, bi, bs);
  };
  for (int k = 0; k < K; ++k) {
    float bv, bs;
    int bi;
    best_left(bv, bi, bs);
    if (bi / VPR == l) taken |= 1u << (bi % VPR);
    if (l == k) { my_w = bs; my_id = bi; }
  }
  if (cutoff_out) {
    // the best choice value left after the K winners: the (K+1)-th of a sorted top-(K+1)
    float bv, bs;
    int bi;
    best_left(bv, bi, bs);
    if (l == 0 && live) cutoff_out[t] = bv;
  }
  if (route_norm) {
    const float sum = row_sum(l < K ? my_w : 0.0f);
    my_w = my_w / (sum + 1e-20f);
  }
  my_w = my_w * route_scale;
  if (l < K && live) {
    weights[static_cast<int64_t>(t) * K + l] = my_w;
    ids[static_cast<int64_t>(t) * K + l] = my_id;
  }
  if (map_out && live) {
    // one-hot routing map of the token, one byte per expert: this lane's VPR experts, four bytes a store
    uint32_t* dst = reinterpret_cast<uint32_t*>(map_out + static_cast<int64_t>(t) * E + e0);
#pragma unroll
    for (int q = 0; q < VPR / 4; ++q) {
      const unsigned b = taken >> (q * 4);
      dst[q] = (b & 1u) | ((b & 2u) << 7) | ((b & 4u) << 14) | ((b & 8u) << 21);
    }
  }
}

// whether select_rows_kernel serves this call
inline bool select_rows_ok(const float* logits, const float* bias, const float* scores, const uint8_t* map,
                           int64_t E, int64_t K, int num_groups, int mode) {
  return mode == MI355_SELECT_TOPK && (num_groups == 0 || (num_groups <= 16 && 16 % num_groups == 0)) && K <= 16 &&
         (E == 64 || E == 128 || E == 256) &&
         reinterpret_cast<uintptr_t>(logits) % 16 == 0 && reinterpret_cast<uintptr_t>(bias) % 16 == 0 &&
         reinterpret_cast<uintptr_t>(scores) % 16 == 0 && reinterpret_cast<uintptr_t>(map) % 4 == 0;
}
template <typename... Args>
void launch_select_rows(int64_t E, int64_t T, hipStream_t s, Args... args) {
  const dim3 grid((unsigned)((T + 15) / 16));
  if (E == 64) hipLaunchKernelGGL(select_rows_kernel<4>, grid, dim3(256), 0, s, args...);
  else if (E == 128) hipLaunchKernelGGL(select_rows_kernel<8>, grid, dim3(256), 0, s, args...);
  else hipLaunchKernelGGL(select_rows_kernel<16>, grid, dim3(256), 0, s, args...);
}

template <int VPL>
__global__ __launch_bounds__(256) void select_bwd_kernel(
    const float* __restrict__ logits, const int64_t* __restrict__ ids,
    const float* __restrict__ dweights, const float* __restrict__ dscores,
    float* __restrict__ dlogits, int T, int E, int K, int score_func, int route_norm,
    float route_scale, int mode) {
  extern __shared__ float lds[];  // per wave: sc[E], ds[E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int t_raw = blockIdx.x * 4 + wave;
  const bool active = t_raw < T;
  const int t = active ? t_raw : T - 1;  // inactive waves shadow the last token, store nothing
  float* sc = lds + static_cast<size_t>(wave) * 2 * E;
  float* ds = sc + E;

  const float* row = logits + static_cast<int64_t>(t) * E;
  float s[VPL];
  float xs[VPL];
  compute_scores<VPL>(row, E, lane, score_func, s, xs);
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + j * kWave;
    if (e < E) {
      sc[e] = s[j];
      ds[e] = dscores ? dscores[static_cast<int64_t>(t) * E + e] : 0.0f;
    }
  }
  __syncthreads();

  if (mode != MI355_SELECT_FIXED && dweights) {
    // lanes 0..K-1 own one selected expert each (K <= 64)
    int id = lane < K ? static_cast<int>(ids[static_cast<int64_t>(t) * K + lane]) : 0;
    id = min(max(id, 0), E - 1);
    const float sk = lane < K ? sc[id] : 0.0f;
    const float dw = lane < K ? dweights[static_cast<int64_t>(t) * K + lane] : 0.0f;
    float g;
    if (route_norm) {
      const float denom = wave_sum_dpp(sk) + 1e-20f;
      const float dot = wave_sum_dpp(dw * sk);
      g = route_scale * (dw / denom - dot / (denom * denom));
    } else {
      g = route_scale * dw;
    }
    // scatter-add into the dense score gradient, serially so a repeated id adds up
    for (int k = 0; k < K; ++k) {
      const int idk = __builtin_amdgcn_readlane(id, k);
      const float gk = lane_f32(g, k);
      if (lane == 0) ds[idk] += gk;
    }
  }
  __syncthreads();

  float d[VPL];
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + j * kWave;
    d[j] = e < E ? ds[e] : 0.0f;
  }
  if (score_func == MI355_SCORE_SOFTMAX) {
    float dot = 0.0f;
#pragma unroll
    for (int j = 0; j < VPL; ++j) dot += (lane + j * kWave < E) ? s[j] * d[j] : 0.0f;
    dot = wave_sum_dpp(dot);
#pragma unroll
    for (int j = 0; j < VPL; ++j) d[j] = s[j] * (d[j] - dot);
  } else if (score_func == MI355_SCORE_SIGMOID) {
#pragma unroll
    for (int j = 0; j < VPL; ++j) d[j] = d[j] * s[j] * (1.0f - s[j]);
  } else {
#pragma unroll
    for (int j = 0; j < VPL; ++j) {
      const int e = lane + j * kWave;
      const float x = e < E ? row[e] : 0.0f;
      const float sig = 1.0f / (1.0f + expf(-x));
      const float dsp = x > 20.0f ? 1.0f : sig;  // d softplus / dx
      d[j] = s[j] > 0.0f ? d[j] * dsp / (2.0f * s[j]) : 0.0f;
    }
  }
#pragma unroll
  for (int j = 0; j < VPL; ++j) {
    const int e = lane + j * kWave;
    if (e < E && active) dlogits[static_cast<int64_t>(t) * E + e] = d[j];
  }
}

int check_router_args(int64_t T, int64_t E, int64_t K) {
  MI355_REQUIRE(T >= 0 && T < (1ll << 31), "router: T=%lld out of range", (long long)T);
  MI355_REQUIRE(E >= 1 && E <= kMaxVPL * kWave, "router: E=%lld must be in [1,%d]", (long long)E,
                kMaxVPL * kWave);
  MI355_REQUIRE(K >= 1 && K <= E, "router: K=%lld must be in [1,E]", (long long)K);
  return MI355_OK;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int64_t mi355_router_gate_fwd_workspace_bytes(int64_t T, int64_t D, int64_t E) {
  return (T >= 0 && D >= 1 && E >= 1 && router_x3_ok(MI355_BF16, MI355_F32, D, E)) ? router_x3_fwd_workspace(T, D, E) : 0;
}

extern "C" int mi355_router_gate_fwd(const void* x, int x_dtype, const void* w, int w_dtype,
                                     const float* logit_bias, float* logits, void* workspace,
                                     int64_t T, int64_t D, int64_t E, void* stream) {
  MI355_REQUIRE(T >= 0 && D >= 1 && E >= 1, "router_gate_fwd: bad shape T=%lld D=%lld E=%lld",
                (long long)T, (long long)D, (long long)E);
  MI355_REQUIRE(T < (1ll << 31) && D < (1ll << 31), "router_gate_fwd: shape exceeds int32");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(x && w && logits, "router_gate_fwd: null pointer");
  // bf16 tokens against fp32 weights: three bf16 MFMAs per product, fp32-exact operands
  if (workspace && router_x3_ok(x_dtype, w_dtype, D, E))
    return router_x3_fwd(x, static_cast<const float*>(w), logit_bias, logits, workspace, T, D, E,
                         as_stream(stream));
  GemmArgs g{};
  g.A = x; g.B = w; g.C = logits; g.bias = logit_bias;
  g.a_rs = D; g.a_cs = 1;
  g.b_rs = 1; g.b_cs = D;  // B(k=d, n=e) = w[e][d]
  g.ldc = E; g.M = (int)T; g.N = (int)E; g.K = (int)D;
  g.mode = GEMM_DENSE; g.ksplit = 1;
  return launch_gemm(g, x_dtype, w_dtype, MI355_F32, gemm_grid_dense(g.M, g.N, 1), as_stream(stream));
}

static int gate_bwd_ksplit(int64_t T, int64_t D, int64_t E) {
  const int64_t tiles = ((E + 63) / 64) * ((D + 63) / 64);
  int64_t split = (1024 + tiles - 1) / tiles;
  const int64_t max_split = (T + 255) / 256;
  if (split > max_split) split = max_split;
  if (split < 1) split = 1;
  if (split > 64) split = 64;
  return (int)split;
}

extern "C" int64_t mi355_router_gate_bwd_workspace_bytes(int64_t T, int64_t D, int64_t E) {
  if (T < 0 || D < 1 || E < 1) return 0;
  const int s = gate_bwd_ksplit(T, D, E);
  const int64_t strided = s > 1 ? (int64_t)s * E * D * 4 : 0;
  const int64_t x3 = router_x3_ok(MI355_BF16, MI355_F32, D, E) ? router_x3_bwd_workspace(T, D, E) : 0;
  return strided > x3 ? strided : x3;
}

extern "C" int mi355_router_gate_bwd(const float* dlogits, const void* x, int x_dtype,
                                     const void* w, int w_dtype, void* dx, void* dw,
                                     void* workspace, int64_t T, int64_t D, int64_t E,
                                     void* stream) {
  MI355_REQUIRE(T >= 0 && D >= 1 && E >= 1 && T < (1ll << 31) && D < (1ll << 31),
                "router_gate_bwd: bad shape");
  hipStream_t s = as_stream(stream);
  if (workspace && router_x3_ok(x_dtype, w_dtype, D, E)) {
    MI355_REQUIRE(dlogits && w && (x || !dw), "router_gate_bwd: null pointer");
    return router_x3_bwd(dlogits, x, static_cast<const float*>(w), dx, static_cast<float*>(dw), workspace, T, D, E, s);
  }
  if (dx && T > 0) {
    GemmArgs g{};
    g.A = dlogits; g.B = w; g.C = dx;
    g.a_rs = E; g.a_cs = 1;
    g.b_rs = D; g.b_cs = 1;  // B(k=e, n=d) = w[e][d]
    g.ldc = D; g.M = (int)T; g.N = (int)D; g.K = (int)E;
    g.mode = GEMM_DENSE; g.ksplit = 1;
    int rc = launch_gemm(g, MI355_F32, w_dtype, x_dtype, gemm_grid_dense(g.M, g.N, 1), s);
    if (rc) return rc;
  }
  if (dw) {
    const int split = gate_bwd_ksplit(T, D, E);
    MI355_REQUIRE(split == 1 || workspace, "router_gate_bwd: workspace required");
    GemmArgs g{};
    g.A = dlogits; g.B = x;
    g.a_rs = 1; g.a_cs = E;  // A(m=e, k=t) = dlogits[t][e]
    g.b_rs = D; g.b_cs = 1;  // B(k=t, n=d) = x[t][d]
    g.ldc = D; g.M = (int)E; g.N = (int)D; g.K = (int)T;
    g.mode = GEMM_DENSE; g.ksplit = split;
    g.C = split > 1 ? workspace : dw;
    int rc = launch_gemm(g, MI355_F32, x_dtype, w_dtype, gemm_grid_dense(g.M, g.N, split), s);
    if (rc) return rc;
    if (split > 1)
      return launch_splitk_reduce(static_cast<const float*>(workspace), dw, w_dtype, E * D, split, s);
  }
  return MI355_OK;
}

#define DISPATCH_VPL(E, ...)                           \
  do {                                                 \
    const int vpl_ = (int)(((E) + 63) / 64);           \
    if (vpl_ <= 1) { constexpr int VPL = 1; __VA_ARGS__; } \
    else if (vpl_ <= 2) { constexpr int VPL = 2; __VA_ARGS__; } \
    else if (vpl_ <= 4) { constexpr int VPL = 4; __VA_ARGS__; } \
    else { constexpr int VPL = 8; __VA_ARGS__; }       \
  } while (0)

extern "C" int mi355_router_select_fwd(const float* logits, const float* expert_bias,
                                       float* weights, int64_t* ids, float* scores_TE,
                                       uint8_t* routing_map_TE, int64_t T, int64_t E, int64_t K,
                                       int score_func, int route_norm, float route_scale, int num_groups,
                                       int num_limited, int select_mode, void* stream) {
  if (int rc = check_router_args(T, E, K)) return rc;
  MI355_REQUIRE(score_func >= 0 && score_func <= 2, "router_select_fwd: unknown score_func %d", score_func);
  MI355_REQUIRE(select_mode >= 0 && select_mode <= 2, "router_select_fwd: unknown select_mode %d", select_mode);
  MI355_REQUIRE(K <= 64, "router_select_fwd: top_k > 64 unsupported");
  if (num_groups > 0) {
    MI355_REQUIRE(num_groups <= 64 && E % num_groups == 0 && E / num_groups >= 2 &&
                      num_limited >= 1 && num_limited <= num_groups &&
                      K <= (int64_t)num_limited * (E / num_groups),
                  "router_select_fwd: bad group config G=%d L=%d", num_groups, num_limited);
  }
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(logits && weights && ids, "router_select_fwd: null pointer");
  if (select_rows_ok(logits, expert_bias, scores_TE, routing_map_TE, E, K, num_groups, select_mode)) {
    launch_select_rows(E, T, as_stream(stream), logits, expert_bias, weights, ids, scores_TE, routing_map_TE,
                       static_cast<float*>(nullptr), (int)T, (int)K, score_func, route_norm, route_scale, num_groups,
                       num_limited);
    return check_launch("router_select_fwd");
  }
  const dim3 grid((unsigned)((T + 3) / 4));
  DISPATCH_VPL(E, hipLaunchKernelGGL(select_fwd_kernel<VPL>, grid, dim3(256), 0, as_stream(stream),
                                     logits, expert_bias, weights, ids, scores_TE, routing_map_TE,
                                     static_cast<float*>(nullptr), (int)T, (int)E, (int)K, score_func,
                                     route_norm, route_scale, num_groups, num_limited, select_mode));
  return check_launch("router_select_fwd");
}

extern "C" int mi355_router_select_cutoff_fwd(const float* logits, const float* expert_bias,
                                              float* weights, int64_t* ids, float* scores_TE,
                                              float* cutoff_T, int64_t T, int64_t E, int64_t K,
                                              int score_func, int route_norm, float route_scale,
                                              void* stream) {
  if (int rc = check_router_args(T, E, K)) return rc;
  MI355_REQUIRE(score_func >= 0 && score_func <= 2, "router_select_cutoff_fwd: unknown score_func %d", score_func);
  MI355_REQUIRE(K <= 64, "router_select_cutoff_fwd: top_k > 64 unsupported");
  MI355_REQUIRE(K < E, "router_select_cutoff_fwd: top_k (%lld) must leave a (K+1)-th expert of %lld",
                (long long)K, (long long)E);
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(logits && weights && ids && cutoff_T, "router_select_cutoff_fwd: null pointer");
  if (select_rows_ok(logits, expert_bias, scores_TE, nullptr, E, K, 0, MI355_SELECT_TOPK) &&
      reinterpret_cast<uintptr_t>(cutoff_T) % 4 == 0) {
    launch_select_rows(E, T, as_stream(stream), logits, expert_bias, weights, ids, scores_TE,
                       static_cast<uint8_t*>(nullptr), cutoff_T, (int)T, (int)K, score_func, route_norm, route_scale, 0, 0);
    return check_launch("router_select_cutoff_fwd");
  }
  const dim3 grid((unsigned)((T + 3) / 4));
  DISPATCH_VPL(E, hipLaunchKernelGGL(select_fwd_kernel<VPL>, grid, dim3(256), 0, as_stream(stream),
                                     logits, expert_bias, weights, ids, scores_TE,
                                     static_cast<uint8_t*>(nullptr), cutoff_T, (int)T,
                                     (int)E, (int)K, score_func, route_norm, route_scale, 0, 0,
                                     MI355_SELECT_TOPK));
  return check_launch("router_select_cutoff_fwd");
}

extern "C" int mi355_router_select_bwd(const float* logits, const int64_t* ids,
                                       const float* dweights, const float* dscores_TE,
                                       float* dlogits, int64_t T, int64_t E, int64_t K,
                                       int score_func, int route_norm, float route_scale,
                                       int select_mode, void* stream) {
  if (int rc = check_router_args(T, E, K)) return rc;
  MI355_REQUIRE(K <= 64, "router_select_bwd: top_k > 64 unsupported");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(logits && ids && dlogits, "router_select_bwd: null pointer");
  const dim3 grid((unsigned)((T + 3) / 4));
  const size_t lds = (size_t)4 * 2 * E * sizeof(float);
  DISPATCH_VPL(E, hipLaunchKernelGGL(select_bwd_kernel<VPL>, grid, dim3(256), lds, as_stream(stream),
                                     logits, ids, dweights, dscores_TE, dlogits, (int)T, (int)E,
                                     (int)K, score_func, route_norm, route_scale, select_mode));
  return check_launch("router_select_bwd");
}
