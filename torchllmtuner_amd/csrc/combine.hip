// Weighted unpermute-combine and its backward (which also yields the router's
// score gradient).  Both are bandwidth kernels: one wavefront per token, 16-byte
// lanes along D, the K row indices and weights held in lanes 0..K-1 and broadcast
// by shuffles.  No atomics: every output element has exactly one writer, so the
// result is deterministic.
#include "common.h"

namespace mi355 {
namespace {

template <typename T>
struct Vec {
  static constexpr int N = 16 / sizeof(T);
  __device__ static void unpack(const uint4& v, float (&f)[N]);
  __device__ static uint4 pack(const float (&f)[N]);
};
template <>
__device__ inline void Vec<float>::unpack(const uint4& v, float (&f)[4]) {
  f[0] = __uint_as_float(v.x); f[1] = __uint_as_float(v.y);
  f[2] = __uint_as_float(v.z); f[3] = __uint_as_float(v.w);
}
template <>
__device__ inline uint4 Vec<float>::pack(const float (&f)[4]) {
  return make_uint4(__float_as_uint(f[0]), __float_as_uint(f[1]), __float_as_uint(f[2]),
                    __float_as_uint(f[3]));
}
template <>
__device__ inline void Vec<uint16_t>::unpack(const uint4& v, float (&f)[8]) {
  f[0] = __uint_as_float(v.x << 16); f[1] = __uint_as_float(v.x & 0xffff0000u);
  f[2] = __uint_as_float(v.y << 16); f[3] = __uint_as_float(v.y & 0xffff0000u);
  f[4] = __uint_as_float(v.z << 16); f[5] = __uint_as_float(v.z & 0xffff0000u);
  f[6] = __uint_as_float(v.w << 16); f[7] = __uint_as_float(v.w & 0xffff0000u);
}
template <>
__device__ inline uint4 Vec<uint16_t>::pack(const float (&f)[8]) {
  return make_uint4(pack_bf16x2(f[0], f[1]), pack_bf16x2(f[2], f[3]), pack_bf16x2(f[4], f[5]),
                    pack_bf16x2(f[6], f[7]));
}

template <typename T>
__device__ __forceinline__ float round_to(float v);
template <>
__device__ __forceinline__ float round_to<float>(float v) { return v; }
template <>
__device__ __forceinline__ float round_to<uint16_t>(float v) { return round_bf16(v); }

// SMALL_K: K <= 8, the eight-row chunk below is the only one
template <typename T, bool SMALL_K>
__global__ __launch_bounds__(256) void combine_fwd_kernel(
    const T* __restrict__ y, const float* __restrict__ weights,
    const int32_t* __restrict__ row_of_slot, T* __restrict__ out, int T_, int D, int K,
    int round_terms) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  const int row = lane < K ? row_of_slot[s0 + lane] : -1;
  const float w = lane < K ? weights[s0 + lane] : 0.0f;
  // ascending-row visiting order (index_add's order): position of each valid slot
  int pos = 0;
  for (int j = 0; j < K; ++j) {
    const int rj = __builtin_amdgcn_readlane(row, j);  // j is wave-uniform: a lane read, not an LDS permute
    pos += (rj >= 0 && (rj < row || (rj == row && j < lane))) ? 1 : 0;
  }
  const int nvalid = __popcll(__ballot(row >= 0));
  // lane p receives the p-th visited slot: every valid lane sends its (row, weight) to lane
  // `pos` (one cross-lane permute each); the others send to lane 63, which is past the last
  // valid position whenever such a lane exists and is not read then
  const int to = (row >= 0 ? pos : 63) << 2;
  int o_row = __builtin_amdgcn_ds_permute(to, row);
  float o_w = __int_as_float(__builtin_amdgcn_ds_permute(to, __float_as_int(w)));
  if (lane >= nvalid) { o_row = -1; o_w = 0.0f; }

  constexpr int V = Vec<T>::N;
  T* dst = out + static_cast<int64_t>(t) * D;
  // Loops are uniform across the wave (shuffles need every lane).
  if (D % V == 0) {
    const int nv = D / V;
    // G vectors per lane and pass (4 KiB of every row per wave) from eight rows at a time, all
    // requested before the first is used: 32 KiB in flight per wave.  Rows and weights are
    // wave-uniform; the terms are still added in visiting order.
    constexpr int G = 4, B = 8;
    auto request = [&](int base, int p0, uint4 (&v)[B][G], float (&ww)[B]) {
#pragma unroll
      for (int j = 0; j < B; ++j) {
        const int p = max(min(p0 + j, nvalid - 1), 0);  // past the end: not loaded, not used
        const int r = __builtin_amdgcn_readlane(o_row, p);  // p is wave-uniform
        ww[j] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(o_w), p));
        const uint4* src = reinterpret_cast<const uint4*>(y + static_cast<int64_t>(max(r, 0)) * D);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int i = base + g * kWave + lane;
          v[j][g] = (p0 + j < nvalid && i < nv) ? load_stream(src + i) : make_uint4(0, 0, 0, 0);
        }
      }
    };
    auto add_terms = [&](float (&a)[V], const uint4& v, float w) {
      float f[V];
      Vec<T>::unpack(v, f);
#pragma unroll
      for (int q = 0; q < V; ++q) {
        const float term = f[q] * w;
        a[q] += round_terms ? round_to<T>(term) : term;
      }
    };
    for (int base = 0; base < nv; base += G * kWave) {
      if constexpr (SMALL_K) {
        // one chunk: each vector is summed and stored on its own (8 live accumulators, not 32,
        // which is what lets three waves share a SIMD)
        uint4 v[B][G];
        float ww[B];
        request(base, 0, v, ww);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          float a[V];
#pragma unroll
          for (int q = 0; q < V; ++q) a[q] = 0.0f;
#pragma unroll
          for (int j = 0; j < B; ++j)
            if (j < nvalid) add_terms(a, v[j][g], ww[j]);
          const int i = base + g * kWave + lane;
          if (i < nv) reinterpret_cast<uint4*>(dst)[i] = Vec<T>::pack(a);
        }
      } else {
        float a[G][V];
#pragma unroll
        for (int g = 0; g < G; ++g)
#pragma unroll
          for (int q = 0; q < V; ++q) a[g][q] = 0.0f;
        for (int p0 = 0; p0 < nvalid; p0 += B) {
          uint4 v[B][G];
          float ww[B];
          request(base, p0, v, ww);
#pragma unroll
          for (int j = 0; j < B; ++j)
            if (p0 + j < nvalid) {
#pragma unroll
              for (int g = 0; g < G; ++g) add_terms(a[g], v[j][g], ww[j]);
            }
        }
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int i = base + g * kWave + lane;
          if (i < nv) reinterpret_cast<uint4*>(dst)[i] = Vec<T>::pack(a[g]);
        }
      }
    }
  } else {
    for (int base = 0; base < D; base += kWave) {
      const int i = base + lane;
      const bool on = i < D;
      float a = 0.0f;
      for (int p = 0; p < nvalid; ++p) {
        const int r = __shfl(o_row, p, kWave);
        const float ww = __shfl(o_w, p, kWave);
        if (!on) continue;
        const float term = load_as_f32(y + static_cast<int64_t>(r) * D + i) * ww;
        a += round_terms ? round_to<T>(term) : term;
      }
      if (on) store_from_f32(dst + i, a);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void combine_bwd_kernel(
    const T* __restrict__ dout, const T* __restrict__ y, const float* __restrict__ weights,
    const int32_t* __restrict__ row_of_slot, const int32_t* __restrict__ slot_of_row,
    const int32_t* __restrict__ total_rows, T* __restrict__ dy, float* __restrict__ dweights,
    int T_, int D, int K, int token_blocks, int row_capacity, int stream_stores) {
  const int lane = threadIdx.x & 63;
  constexpr int V = Vec<T>::N;
  if (static_cast<int>(blockIdx.x) >= token_blocks) {
    // padding rows of dy get zeros
    const int r = (blockIdx.x - token_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= row_capacity || r >= *total_rows || slot_of_row[r] >= 0) return;
    T* dst = dy + static_cast<int64_t>(r) * D;
    for (int i = lane; i < D; i += kWave) dst[i] = T(0);
    return;
  }
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  const int row = lane < K ? row_of_slot[s0 + lane] : -1;
  const float w = lane < K ? weights[s0 + lane] : 0.0f;
  const T* g = dout + static_cast<int64_t>(t) * D;
  float my_dot = 0.0f;  // lane k keeps slot k's dot product
  if (D % V == 0) {
    // The token's gradient row is read ONCE per pass of G vectors per lane (4 KiB of the row per
    // wave: all of it at D = 2048 bf16) and kept in registers while the K expert rows stream by;
    // re-reading it per slot fetched it K times from wherever it had gone meanwhile.
    const int nv = D / V;
    constexpr int G = 4;
    for (int base = 0; base < nv; base += G * kWave) {
      float gf[G][V];
#pragma unroll
      for (int q = 0; q < G; ++q) {
        const int i = base + q * kWave + lane;
        Vec<T>::unpack(i < nv ? reinterpret_cast<const uint4*>(g)[i] : make_uint4(0, 0, 0, 0), gf[q]);
      }
      for (int k = 0; k < K; ++k) {
        const int r = __shfl(row, k, kWave);
        const float ww = __shfl(w, k, kWave);
        if (r < 0) continue;
        const uint4* yr = reinterpret_cast<const uint4*>(y + static_cast<int64_t>(r) * D);
        uint4* dr = reinterpret_cast<uint4*>(dy + static_cast<int64_t>(r) * D);
        uint4 yv[G];
#pragma unroll
        for (int q = 0; q < G; ++q) {
          const int i = base + q * kWave + lane;
          yv[q] = i < nv ? load_stream(yr + i) : make_uint4(0, 0, 0, 0);
        }
        float dot = 0.0f;
#pragma unroll
        for (int q = 0; q < G; ++q) {
          const int i = base + q * kWave + lane;
          float yf[V], o[V];
          Vec<T>::unpack(yv[q], yf);
#pragma unroll
          for (int c = 0; c < V; ++c) {
            dot += yf[c] * gf[q][c];
            o[c] = gf[q][c] * ww;
          }
          if (i < nv) {
            if (stream_stores) store_stream(dr + i, Vec<T>::pack(o));
            else dr[i] = Vec<T>::pack(o);
          }
        }
        dot = wave_sum(dot);
        if (lane == k) my_dot += dot;
      }
    }
  } else {
    for (int k = 0; k < K; ++k) {
      const int r = __shfl(row, k, kWave);
      const float ww = __shfl(w, k, kWave);
      if (r < 0) continue;
      const T* yr = y + static_cast<int64_t>(r) * D;
      T* dr = dy + static_cast<int64_t>(r) * D;
      float dot = 0.0f;
      for (int i = lane; i < D; i += kWave) {
        const float gv = load_as_f32(g + i);
        dot += load_as_f32(yr + i) * gv;
        store_from_f32(dr + i, gv * ww);
      }
      dot = wave_sum(dot);
      if (lane == k) my_dot = dot;
    }
  }
  if (lane < K && dweights) dweights[s0 + lane] = my_dot;
}

// ---- fp64 rows: every product and sum in fp64 (the scores stay fp32 and are widened), one wave
// per token, lanes along D; the terms are added in ascending row order like the kernels above
__global__ __launch_bounds__(256) void combine_fwd_f64_kernel(
    const double* __restrict__ y, const float* __restrict__ weights, const int32_t* __restrict__ row_of_slot,
    double* __restrict__ out, int T_, int D, int K) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  const int row = lane < K ? row_of_slot[s0 + lane] : -1;
  const float w = lane < K ? weights[s0 + lane] : 0.0f;
  int pos = 0;
  for (int j = 0; j < K; ++j) {
    const int rj = __shfl(row, j, kWave);
    pos += (rj >= 0 && (rj < row || (rj == row && j < lane))) ? 1 : 0;
  }
  const int nvalid = __popcll(__ballot(row >= 0));
  const int to = (row >= 0 ? pos : 63) << 2;
  int o_row = __builtin_amdgcn_ds_permute(to, row);
  float o_w = __int_as_float(__builtin_amdgcn_ds_permute(to, __float_as_int(w)));
  if (lane >= nvalid) { o_row = -1; o_w = 0.0f; }
  double* dst = out + static_cast<int64_t>(t) * D;
  for (int base = 0; base < D; base += kWave) {  // uniform trip count: the shuffles need every lane
    const int i = base + lane;
    double a = 0.0;
    for (int p = 0; p < nvalid; ++p) {
      const int r = __shfl(o_row, p, kWave);
      const double ww = static_cast<double>(__shfl(o_w, p, kWave));
      if (i < D) a += y[static_cast<int64_t>(r) * D + i] * ww;
    }
    if (i < D) dst[i] = a;
  }
}

__global__ __launch_bounds__(256) void combine_bwd_f64_kernel(
    const double* __restrict__ dout, const double* __restrict__ y, const float* __restrict__ weights,
    const int32_t* __restrict__ row_of_slot, const int32_t* __restrict__ slot_of_row,
    const int32_t* __restrict__ total_rows, double* __restrict__ dy, float* __restrict__ dweights, int T_, int D,
    int K, int token_blocks, int row_capacity) {
  const int lane = threadIdx.x & 63;
  if (static_cast<int>(blockIdx.x) >= token_blocks) {
    const int r = (blockIdx.x - token_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= row_capacity || r >= *total_rows || slot_of_row[r] >= 0) return;
    double* dst = dy + static_cast<int64_t>(r) * D;
    for (int i = lane; i < D; i += kWave) dst[i] = 0.0;
    return;
  }
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  const double* g = dout + static_cast<int64_t>(t) * D;
  for (int k = 0; k < K; ++k) {
    const int r = row_of_slot[s0 + k];  // wave-uniform
    if (r < 0) {
      if (lane == 0 && dweights) dweights[s0 + k] = 0.0f;
      continue;
    }
    const double ww = static_cast<double>(weights[s0 + k]);
    const double* yr = y + static_cast<int64_t>(r) * D;
    double* dr = dy + static_cast<int64_t>(r) * D;
    double dot = 0.0;
    for (int i = lane; i < D; i += kWave) {
      const double gv = g[i];
      dot += yr[i] * gv;
      dr[i] = gv * ww;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) dot += __shfl_xor(dot, o, kWave);
    if (lane == 0 && dweights) dweights[s0 + k] = static_cast<float>(dot);
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_combine_fwd(const void* y, int dtype, const float* weights,
                                 const int32_t* row_of_slot, void* out, int64_t T, int64_t D,
                                 int64_t K, int round_terms, void* stream) {
  MI355_REQUIRE(T >= 0 && D >= 1 && K >= 1 && K <= 64 && T < (1ll << 31) && D < (1ll << 31),
                "combine_fwd: bad shape (K must be <= 64)");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(weights && row_of_slot && out, "combine_fwd: null pointer");
  const dim3 grid((unsigned)((T + 3) / 4));
  auto launch = [&](auto kernel, auto* yp, auto* op) {
    hipLaunchKernelGGL(kernel, grid, dim3(256), 0, as_stream(stream), yp, weights, row_of_slot, op, (int)T, (int)D,
                       (int)K, round_terms);
  };
  if (dtype == MI355_F32) {
    if (K <= 8) launch(combine_fwd_kernel<float, true>, static_cast<const float*>(y), static_cast<float*>(out));
    else launch(combine_fwd_kernel<float, false>, static_cast<const float*>(y), static_cast<float*>(out));
  } else if (dtype == MI355_BF16) {
    if (K <= 8) launch(combine_fwd_kernel<uint16_t, true>, static_cast<const uint16_t*>(y), static_cast<uint16_t*>(out));
    else launch(combine_fwd_kernel<uint16_t, false>, static_cast<const uint16_t*>(y), static_cast<uint16_t*>(out));
  } else if (dtype == MI355_F64) {
    hipLaunchKernelGGL(combine_fwd_f64_kernel, grid, dim3(256), 0, as_stream(stream), static_cast<const double*>(y),
                       weights, row_of_slot, static_cast<double*>(out), (int)T, (int)D, (int)K);
  } else
    return fail(MI355_EINVAL, "combine_fwd: unknown dtype %d", dtype);
  return check_launch("combine_fwd");
}

extern "C" int mi355_combine_bwd(const void* dout, const void* y, int dtype, const float* weights,
                                 const int32_t* row_of_slot, const int32_t* slot_of_row,
                                 const int32_t* total_rows, void* dy, float* dweights, int64_t T,
                                 int64_t D, int64_t K, int64_t row_capacity, void* stream) {
  MI355_REQUIRE(T >= 0 && D >= 1 && K >= 1 && K <= 64 && T < (1ll << 31) && D < (1ll << 31) &&
                    row_capacity >= 0 && row_capacity < (1ll << 31),
                "combine_bwd: bad shape (K must be <= 64)");
  const int token_blocks = (int)((T + 3) / 4);
  const int pad_blocks = slot_of_row ? (int)((row_capacity + 3) / 4) : 0;
  if (token_blocks + pad_blocks == 0) return MI355_OK;
  MI355_REQUIRE(T == 0 || (dout && weights && row_of_slot && dy), "combine_bwd: null pointer");
  MI355_REQUIRE(!slot_of_row || total_rows, "combine_bwd: total_rows required with slot_of_row");
  const dim3 grid((unsigned)(token_blocks + pad_blocks));
  // dy larger than the 256 MiB memory-side cache is written with non-temporal stores (as the
  // row scatter of the forward permutation does)
  const int stream_stores = row_capacity * D * (dtype == MI355_F32 ? 4 : 2) > (256ll << 20);
  if (dtype == MI355_F32)
    hipLaunchKernelGGL(combine_bwd_kernel<float>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const float*>(dout), static_cast<const float*>(y), weights,
                       row_of_slot, slot_of_row, total_rows, static_cast<float*>(dy), dweights,
                       (int)T, (int)D, (int)K, token_blocks, (int)row_capacity, stream_stores);
  else if (dtype == MI355_BF16)
    hipLaunchKernelGGL(combine_bwd_kernel<uint16_t>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t*>(dout), static_cast<const uint16_t*>(y), weights,
                       row_of_slot, slot_of_row, total_rows, static_cast<uint16_t*>(dy), dweights,
                       (int)T, (int)D, (int)K, token_blocks, (int)row_capacity, stream_stores);
  else if (dtype == MI355_F64)
    hipLaunchKernelGGL(combine_bwd_f64_kernel, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const double*>(dout), static_cast<const double*>(y), weights, row_of_slot,
                       slot_of_row, total_rows, static_cast<double*>(dy), dweights, (int)T, (int)D, (int)K,
                       token_blocks, (int)row_capacity);
  else
    return fail(MI355_EINVAL, "combine_bwd: unknown dtype %d", dtype);
  return check_launch("combine_bwd");
}

// ---- the two small ends of the backward that folds the combine into the expert kernels --
namespace mi355 {
namespace {

__global__ __launch_bounds__(256) void row_scale_kernel(const float* __restrict__ weights,
                                                        const int32_t* __restrict__ slot_of_row,
                                                        float* __restrict__ row_scale, int rows, int slots) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= rows) return;
  const int slot = slot_of_row[r];
  row_scale[r] = (slot >= 0 && slot < slots) ? weights[slot] : 0.0f;
}

__global__ __launch_bounds__(256) void scores_bwd_kernel(const float* __restrict__ partial, int pieces,
                                                         const int32_t* __restrict__ row_of_slot,
                                                         float* __restrict__ dweights, int slots, int rows) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= slots) return;
  const int row = row_of_slot[i];
  float acc = 0.0f;
  if (row >= 0 && row < rows) {
    const float* src = partial + static_cast<int64_t>(row) * pieces;
    for (int s = 0; s < pieces; ++s) acc += src[s];  // fixed order: the same bits every run
  }
  dweights[i] = acc;
}

}  // namespace
}  // namespace mi355

extern "C" int mi355_combine_row_scale(const float* weights_TK, const int32_t* slot_of_row, float* row_scale,
                                       int64_t T, int64_t K, int64_t row_capacity, void* stream) {
  using namespace mi355;
  MI355_REQUIRE(T >= 0 && K >= 1 && T * K < (1ll << 31) && row_capacity >= 0 && row_capacity < (1ll << 31),
                "combine_row_scale: bad shape");
  if (row_capacity == 0) return MI355_OK;
  MI355_REQUIRE(slot_of_row && row_scale && (weights_TK || T == 0), "combine_row_scale: null pointer");
  hipLaunchKernelGGL(row_scale_kernel, dim3((unsigned)((row_capacity + 255) / 256)), dim3(256), 0,
                     as_stream(stream), weights_TK, slot_of_row, row_scale, (int)row_capacity, (int)(T * K));
  return check_launch("combine_row_scale");
}

extern "C" int mi355_combine_scores_bwd(const float* dot_partial, int64_t pieces, const int32_t* row_of_slot,
                                        float* dweights_TK, int64_t T, int64_t K, int64_t row_capacity,
                                        void* stream) {
  using namespace mi355;
  MI355_REQUIRE(T >= 0 && K >= 1 && T * K < (1ll << 31) && pieces >= 1 && pieces <= 4096 && row_capacity >= 0 &&
                    row_capacity < (1ll << 31),
                "combine_scores_bwd: bad shape");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(row_of_slot && dweights_TK && (dot_partial || row_capacity == 0), "combine_scores_bwd: null pointer");
  hipLaunchKernelGGL(scores_bwd_kernel, dim3((unsigned)((T * K + 255) / 256)), dim3(256), 0, as_stream(stream),
                     dot_partial, (int)pieces, row_of_slot, dweights_TK, (int)(T * K), (int)row_capacity);
  return check_launch("combine_scores_bwd");
}

