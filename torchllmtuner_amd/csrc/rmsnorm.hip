// RMS normalisation over the last axis and its backward: the `rms_norm` entry of the
// reference's kernel registry (llmtuner/kernel/ops/rms_norm.py:10-31; reference math
// llmtuner/kernel/cpu/basic.py:17-25 = torch.nn.functional.rms_norm).
//
//   r_t = rsqrt(mean_d x[t][d]^2 + eps)      y[t][d] = round((x[t][d] * r_t) * w[d])
//
// with everything in fp32 and ONE rounding to the storage type at the end, which is what
// torch's CPU routine does for bf16 inputs.  Backward, with g = dy * w and xh = x * r:
//   dx[t][d] = r_t * (g[t][d] - xh[t][d] * mean_d(g[t][.] * xh[t][.]))
//   dw[d]    = sum_t dy[t][d] * xh[t][d]
// HBM-bound: one wavefront per row for y and dx (16-byte lanes, the second pass over the
// row comes from cache); dw as per-workgroup column sums over a run of rows, combined by a
// second kernel in a fixed order (no atomics, deterministic).
#include <algorithm>
#include <initializer_list>
#include <type_traits>

#include "common.h"

namespace mi355 {
namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

// N consecutive elements as floats; N = 16 bytes' worth uses one 16-byte access
template <typename T, int N>
struct Pack;
template <>
struct Pack<float, 1> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[1]) { v[0] = *p; }
  static __device__ __forceinline__ void store(float* p, const float (&v)[1]) { *p = v[0]; }
};
template <>
struct Pack<float, 4> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[4]) {
    const float4 q = *reinterpret_cast<const float4*>(p);
    v[0] = q.x; v[1] = q.y; v[2] = q.z; v[3] = q.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[4]) {
    *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
  }
};
template <>
struct Pack<uint16_t, 1> {
  static __device__ __forceinline__ void load(const uint16_t* p, float (&v)[1]) { v[0] = bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&v)[1]) { *p = f32_to_bf16(v[0]); }
};
template <>
struct Pack<uint16_t, 8> {
  static __device__ __forceinline__ void load(const uint16_t* p, float (&v)[8]) {
    const u32x4 q = *reinterpret_cast<const u32x4*>(p);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = __uint_as_float(q[j] << 16);
      v[2 * j + 1] = __uint_as_float(q[j] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(uint16_t* p, const float (&v)[8]) {
    u32x4 q;
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
    *reinterpret_cast<u32x4*>(p) = q;
  }
};
template <typename T>
constexpr int kVec = 16 / sizeof(T);

template <typename T, int N>
__device__ __forceinline__ float row_sumsq(const T* xr, int D, int lane) {
  float ss = 0.0f;
  for (int i = lane * N; i < D; i += kWave * N) {
    float v[N];
    Pack<T, N>::load(xr + i, v);
#pragma unroll
    for (int j = 0; j < N; ++j) ss += v[j] * v[j];
  }
  return ss;
}

template <typename T, int N>
__device__ __forceinline__ void row_scale(const T* xr, const T* w, T* yr, float r, int D, int lane) {
  for (int i = lane * N; i < D; i += kWave * N) {
    float v[N], g[N], o[N];
    Pack<T, N>::load(xr + i, v);
    Pack<T, N>::load(w + i, g);
#pragma unroll
    for (int j = 0; j < N; ++j) o[j] = (v[j] * r) * g[j];
    Pack<T, N>::store(yr + i, o);
  }
}

// vec: rows start on 16-byte boundaries (D a multiple of 16 bytes' worth, aligned bases)
template <typename T>
__global__ __launch_bounds__(256) void rms_fwd_kernel(const T* __restrict__ x, const T* __restrict__ w,
                                                      T* __restrict__ y, float* __restrict__ rstd, int rows,
                                                      int D, float eps, int vec) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const T* xr = x + static_cast<int64_t>(row) * D;
  T* yr = y + static_cast<int64_t>(row) * D;
  const float ss = wave_sum(vec ? row_sumsq<T, kVec<T>>(xr, D, lane) : row_sumsq<T, 1>(xr, D, lane));
  const float r = 1.0f / sqrtf(ss / static_cast<float>(D) + eps);
  if (vec) row_scale<T, kVec<T>>(xr, w, yr, r, D, lane); else row_scale<T, 1>(xr, w, yr, r, D, lane);
  if (lane == 0 && rstd) rstd[row] = r;
}

template <typename T, int N>
__device__ __forceinline__ float row_dot(const T* dyr, const T* xr, const T* w, float r, int D, int lane) {
  float dot = 0.0f;
  for (int i = lane * N; i < D; i += kWave * N) {
    float a[N], b[N], g[N];
    Pack<T, N>::load(dyr + i, a);
    Pack<T, N>::load(xr + i, b);
    Pack<T, N>::load(w + i, g);
#pragma unroll
    for (int j = 0; j < N; ++j) dot += (a[j] * g[j]) * (b[j] * r);
  }
  return dot;
}

template <typename T, int N>
__device__ __forceinline__ void row_dx(const T* dyr, const T* xr, const T* w, T* dxr, float r, float c, int D,
                                       int lane) {
  for (int i = lane * N; i < D; i += kWave * N) {
    float a[N], b[N], g[N], o[N];
    Pack<T, N>::load(dyr + i, a);
    Pack<T, N>::load(xr + i, b);
    Pack<T, N>::load(w + i, g);
#pragma unroll
    for (int j = 0; j < N; ++j) o[j] = r * (a[j] * g[j] - (b[j] * r) * c);
    Pack<T, N>::store(dxr + i, o);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rms_dx_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                     const T* __restrict__ w, const float* __restrict__ rstd,
                                                     T* __restrict__ dx, int rows, int D, int vec) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= rows) return;
  const int64_t o = static_cast<int64_t>(row) * D;
  const float r = rstd[row];
  const float dot = vec ? row_dot<T, kVec<T>>(dy + o, x + o, w, r, D, lane) : row_dot<T, 1>(dy + o, x + o, w, r, D, lane);
  const float c = wave_sum(dot) / static_cast<float>(D);
  if (vec) row_dx<T, kVec<T>>(dy + o, x + o, w, dx + o, r, c, D, lane);
  else row_dx<T, 1>(dy + o, x + o, w, dx + o, r, c, D, lane);
}

// dx and the column sums of dweight in one pass over dy and x: a workgroup walks a run of
// rows, one wavefront per row; a lane keeps the dweight partial sums of the columns it owns
// in registers across its rows (ITER 16-byte groups per lane), the four waves add theirs up
// through LDS at the end and the workgroup writes one row of partial sums.
constexpr int kFusedBlocks = 2048;  // at most; 512 until a workgroup would get more than 32 rows

template <typename T, int ITER>
__global__ __launch_bounds__(256) void rms_bwd_fused_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                            const T* __restrict__ w,
                                                            const float* __restrict__ rstd, T* __restrict__ dx,
                                                            float* __restrict__ partial, int rows, int D,
                                                            int rows_per_block) {
  constexpr int N = kVec<T>;
  extern __shared__ float colsum[];  // [D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float acc[ITER][N];
#pragma unroll
  for (int k = 0; k < ITER; ++k)
#pragma unroll
    for (int j = 0; j < N; ++j) acc[k][j] = 0.0f;
  const int r0 = blockIdx.x * rows_per_block;
  const int r1 = min(r0 + rows_per_block, rows);
  for (int row = r0 + wave; row < r1; row += 4) {
    const int64_t o = static_cast<int64_t>(row) * D;
    const float r = rstd[row];
    const float c = wave_sum(row_dot<T, N>(dy + o, x + o, w, r, D, lane)) / static_cast<float>(D);
#pragma unroll
    for (int k = 0; k < ITER; ++k) {
      const int i = (k * kWave + lane) * N;
      if (i < D) {
        float a[N], b[N], g[N], out[N];
        Pack<T, N>::load(dy + o + i, a);
        Pack<T, N>::load(x + o + i, b);
        Pack<T, N>::load(w + i, g);
#pragma unroll
        for (int j = 0; j < N; ++j) {
          const float xh = b[j] * r;
          out[j] = r * (a[j] * g[j] - xh * c);
          acc[k][j] += a[j] * xh;
        }
        if (dx) Pack<T, N>::store(dx + o + i, out);
      }
    }
  }
  for (int turn = 0; turn < 4; ++turn) {
    if (wave == turn) {
#pragma unroll
      for (int k = 0; k < ITER; ++k) {
        const int i = (k * kWave + lane) * N;
        if (i < D) {
#pragma unroll
          for (int j = 0; j < N; ++j) colsum[i + j] = turn == 0 ? acc[k][j] : colsum[i + j] + acc[k][j];
        }
      }
    }
    __syncthreads();
  }
  for (int d = threadIdx.x; d < D; d += 256) partial[static_cast<int64_t>(blockIdx.x) * D + d] = colsum[d];
}

// 16 bytes of T as N floats and back
template <typename T, int N>
__device__ __forceinline__ void unpack16(const u32x4& q, float (&v)[N]) {
  if constexpr (std::is_same<T, float>::value) {
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = __uint_as_float(q[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      v[2 * j] = __uint_as_float(q[j] << 16);
      v[2 * j + 1] = __uint_as_float(q[j] & 0xffff0000u);
    }
  }
}
template <typename T, int N>
__device__ __forceinline__ u32x4 pack16(const float (&v)[N]) {
  u32x4 q;
  if constexpr (std::is_same<T, float>::value) {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = __float_as_uint(v[j]);
  } else {
#pragma unroll
    for (int j = 0; j < 4; ++j) q[j] = pack_bf16x2(v[2 * j], v[2 * j + 1]);
  }
  return q;
}

// The same pass for rows of at most 4 x 64 sixteen-byte groups (2048 bf16 or 1024 fp32 columns): a
// wave holds its row of dy and x in registers, so the row is read from memory once (the kernel
// above reads it for the row's dot product and again, from cache, for dx), the weights stay in
// registers across the rows, and the next row of the wave is requested before the current one is
// reduced -- with one row in flight per wave the kernel waited out a memory round trip per row.
template <typename T, int ITER>
__global__ __launch_bounds__(256) void rms_bwd_rows_in_registers_kernel(
    const T* __restrict__ dy, const T* __restrict__ x, const T* __restrict__ w, const float* __restrict__ rstd,
    T* __restrict__ dx, float* __restrict__ partial, int rows, int D, int rows_per_block) {
  constexpr int N = kVec<T>;
  extern __shared__ float colsum[];  // [D]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float acc[ITER][N], g[ITER][N];
  const u32x4 zero = {0, 0, 0, 0};
#pragma unroll
  for (int k = 0; k < ITER; ++k) {
    const int i = (k * kWave + lane) * N;
    u32x4 q = zero;
    if (i < D) q = *reinterpret_cast<const u32x4*>(w + i);
    unpack16<T, N>(q, g[k]);
#pragma unroll
    for (int j = 0; j < N; ++j) acc[k][j] = 0.0f;
  }
  const int r0 = blockIdx.x * rows_per_block;
  const int r1 = min(r0 + rows_per_block, rows);
  u32x4 cdy[ITER], cx[ITER];
  auto fetch = [&](int row, u32x4 (&a)[ITER], u32x4 (&b)[ITER]) {
    const int64_t o = static_cast<int64_t>(row) * D;
#pragma unroll
    for (int k = 0; k < ITER; ++k) {
      const int i = (k * kWave + lane) * N;
      a[k] = zero;
      b[k] = zero;
      if (i < D) {
        a[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(dy + o + i));
        b[k] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(x + o + i));
      }
    }
  };
  int row = r0 + wave;
  if (row < r1) fetch(row, cdy, cx);
  for (; row < r1; row += 4) {
    u32x4 ndy[ITER], nx[ITER];
    const bool more = row + 4 < r1;
    if (more) fetch(row + 4, ndy, nx);
    const float r = rstd[row];
    float dot = 0.0f;
#pragma unroll
    for (int k = 0; k < ITER; ++k) {
      float a[N], b[N];
      unpack16<T, N>(cdy[k], a);
      unpack16<T, N>(cx[k], b);
#pragma unroll
      for (int j = 0; j < N; ++j) dot += (a[j] * g[k][j]) * (b[j] * r);
    }
    const float c = wave_sum(dot) / static_cast<float>(D);
    const int64_t o = static_cast<int64_t>(row) * D;
#pragma unroll
    for (int k = 0; k < ITER; ++k) {
      const int i = (k * kWave + lane) * N;
      float a[N], b[N], out[N];
      unpack16<T, N>(cdy[k], a);
      unpack16<T, N>(cx[k], b);
#pragma unroll
      for (int j = 0; j < N; ++j) {
        const float xh = b[j] * r;
        out[j] = r * (a[j] * g[k][j] - xh * c);
        acc[k][j] += a[j] * xh;
      }
      if (dx && i < D) *reinterpret_cast<u32x4*>(dx + o + i) = pack16<T, N>(out);
    }
    if (more) {
#pragma unroll
      for (int k = 0; k < ITER; ++k) {
        cdy[k] = ndy[k];
        cx[k] = nx[k];
      }
    }
  }
  for (int turn = 0; turn < 4; ++turn) {
    if (wave == turn) {
#pragma unroll
      for (int k = 0; k < ITER; ++k) {
        const int i = (k * kWave + lane) * N;
        if (i < D) {
#pragma unroll
          for (int j = 0; j < N; ++j) colsum[i + j] = turn == 0 ? acc[k][j] : colsum[i + j] + acc[k][j];
        }
      }
    }
    __syncthreads();
  }
  for (int d = threadIdx.x; d < D; d += 256) partial[static_cast<int64_t>(blockIdx.x) * D + d] = colsum[d];
}

// rows per workgroup of the column sums: 64, more once that would exceed 4096 workgroups
__host__ __device__ inline int64_t dw_rows_per_chunk(int64_t rows) {
  const int64_t per = (rows + 4095) / 4096;
  return per < 64 ? 64 : per;
}

// partial[chunk][d] = sum over the chunk's rows of dy * x * r
template <typename T>
__global__ __launch_bounds__(256) void rms_dw_partial_kernel(const T* __restrict__ dy, const T* __restrict__ x,
                                                             const float* __restrict__ rstd,
                                                             float* __restrict__ partial, int rows, int D,
                                                             int per) {
  const int d = blockIdx.x * 256 + threadIdx.x;
  const int r0 = blockIdx.y * per;
  const int r1 = min(r0 + per, rows);
  if (d >= D) return;
  float acc = 0.0f;
  for (int row = r0; row < r1; ++row) {
    const int64_t o = static_cast<int64_t>(row) * D + d;
    float a[1], b[1];
    Pack<T, 1>::load(dy + o, a);
    Pack<T, 1>::load(x + o, b);
    acc += a[0] * (b[0] * rstd[row]);
  }
  partial[static_cast<int64_t>(blockIdx.y) * D + d] = acc;
}

// dw[d] = sum over the chunks of partial[chunk][d]: 16 columns x 16 slices per workgroup, slice
// s adds chunks s, s+16, ... (independent loads, several in flight), the slices are then
// added in order -- a fixed summation tree.
template <typename T>
__global__ __launch_bounds__(256) void rms_dw_final_kernel(const float* __restrict__ partial, T* __restrict__ dw,
                                                           int chunks, int D) {
  __shared__ float part[16][17];
  const int col = threadIdx.x & 15, slice = threadIdx.x >> 4;
  const int d = blockIdx.x * 16 + col;
  float acc = 0.0f;
  if (d < D) {
#pragma unroll 8
    for (int c = slice; c < chunks; c += 16) acc += partial[static_cast<int64_t>(c) * D + d];
  }
  part[slice][col] = acc;
  __syncthreads();
  if (slice == 0 && d < D) {
    float total = 0.0f;
#pragma unroll
    for (int k = 0; k < 16; ++k) total += part[k][col];
    const float out[1] = {total};
    Pack<T, 1>::store(dw + d, out);
  }
}

int rows_are_16_byte_aligned(int64_t D, int dtype, std::initializer_list<const void*> ptrs) {
  const int64_t per16 = dtype == MI355_F32 ? 4 : 8;
  if (D % per16 != 0) return 0;
  for (const void* p : ptrs)
    if (reinterpret_cast<uintptr_t>(p) % 16 != 0) return 0;
  return 1;
}

int check_shape(const char* what, int64_t rows, int64_t D, int dtype) {
  MI355_REQUIRE(dtype == MI355_F32 || dtype == MI355_BF16, "%s: dtype %d is neither fp32 nor bf16", what, dtype);
  MI355_REQUIRE(rows >= 0 && rows < (1ll << 31) && D >= 1 && D < (1ll << 31), "%s: bad shape rows=%lld D=%lld", what,
                (long long)rows, (long long)D);
  return MI355_OK;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int mi355_rms_norm_fwd(const void* x, const void* weight, int dtype, void* y, float* rstd,
                                  int64_t rows, int64_t D, float epsilon, void* stream) {
  if (int rc = check_shape("rms_norm_fwd", rows, D, dtype)) return rc;
  MI355_REQUIRE(epsilon >= 0.0f && epsilon < INFINITY, "rms_norm_fwd: epsilon must be finite and nonnegative");
  if (rows == 0) return MI355_OK;
  MI355_REQUIRE(x && weight && y, "rms_norm_fwd: null pointer");
  const dim3 grid((unsigned)((rows + 3) / 4));
  const int vec = rows_are_16_byte_aligned(D, dtype, {x, weight, y});
  if (dtype == MI355_F32)
    hipLaunchKernelGGL(rms_fwd_kernel<float>, grid, dim3(256), 0, as_stream(stream), static_cast<const float*>(x),
                       static_cast<const float*>(weight), static_cast<float*>(y), rstd, (int)rows, (int)D, epsilon,
                       vec);
  else
    hipLaunchKernelGGL(rms_fwd_kernel<uint16_t>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t*>(x), static_cast<const uint16_t*>(weight),
                       static_cast<uint16_t*>(y), rstd, (int)rows, (int)D, epsilon, vec);
  return check_launch("rms_norm_fwd");
}

extern "C" int64_t mi355_rms_norm_bwd_workspace_bytes(int64_t rows, int64_t D) {
  if (rows < 0 || D < 1) return 0;
  const int64_t per = dw_rows_per_chunk(rows);
  return std::max<int64_t>((rows + per - 1) / per, kFusedBlocks) * D * 4;
}

extern "C" int mi355_rms_norm_bwd(const void* dy, const void* x, const void* weight, const float* rstd,
                                  int dtype, void* dx, void* dweight, void* workspace, int64_t rows,
                                  int64_t D, void* stream) {
  if (int rc = check_shape("rms_norm_bwd", rows, D, dtype)) return rc;
  MI355_REQUIRE(rows == 0 || (dy && x && weight && rstd), "rms_norm_bwd: null pointer");
  MI355_REQUIRE(!dweight || rows == 0 || workspace, "rms_norm_bwd: workspace required for dweight");
  hipStream_t s = as_stream(stream);
  const int per = (int)dw_rows_per_chunk(rows);
  const int chunks = (int)((rows + per - 1) / per);
  const dim3 rgrid((unsigned)((rows + 3) / 4));
  const dim3 cgrid((unsigned)((D + 255) / 256), (unsigned)std::max(chunks, 1));
  const dim3 fgrid((unsigned)((D + 15) / 16));
  auto run = [&](auto tag) {
    using T = decltype(tag);
    // one pass for both when rows are 16-byte aligned and a lane's columns fit in registers
    constexpr int N = 16 / sizeof(T);
    const int64_t groups = (D / N + kWave - 1) / kWave;  // 16-byte groups per lane
    if (dweight && rows > 0 && groups <= 16 && D * 4 <= 64 * 1024 &&
        rows_are_16_byte_aligned(D, dtype, {dy, x, weight, dx})) {
      const int blocks = (int)std::min<int64_t>(std::min<int64_t>(kFusedBlocks, std::max<int64_t>(512, rows / 32)),
                                                (rows + 3) / 4);
      const int rpb = (int)((rows + blocks - 1) / blocks);
      const int used = (int)((rows + rpb - 1) / rpb);
      auto launch = [&](auto iter) {
        constexpr int ITER = decltype(iter)::value;
        if constexpr (ITER <= 4) {
          hipLaunchKernelGGL((rms_bwd_rows_in_registers_kernel<T, ITER>), dim3(used), dim3(256), (size_t)D * 4, s,
                             static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(weight), rstd,
                             static_cast<T*>(dx), static_cast<float*>(workspace), (int)rows, (int)D, rpb);
          return;
        }
        hipLaunchKernelGGL((rms_bwd_fused_kernel<T, ITER>), dim3(used), dim3(256), (size_t)D * 4, s,
                           static_cast<const T*>(dy), static_cast<const T*>(x), static_cast<const T*>(weight), rstd,
                           static_cast<T*>(dx), static_cast<float*>(workspace), (int)rows, (int)D, rpb);
      };
      if (groups <= 1) launch(std::integral_constant<int, 1>{});
      else if (groups <= 2) launch(std::integral_constant<int, 2>{});
      else if (groups <= 4) launch(std::integral_constant<int, 4>{});
      else if (groups <= 8) launch(std::integral_constant<int, 8>{});
      else launch(std::integral_constant<int, 16>{});
      hipLaunchKernelGGL(rms_dw_final_kernel<T>, fgrid, dim3(256), 0, s, static_cast<const float*>(workspace),
                         static_cast<T*>(dweight), used, (int)D);
      return;
    }
    if (dx && rows > 0)
      hipLaunchKernelGGL(rms_dx_kernel<T>, rgrid, dim3(256), 0, s, static_cast<const T*>(dy),
                         static_cast<const T*>(x), static_cast<const T*>(weight), rstd, static_cast<T*>(dx),
                         (int)rows, (int)D, rows_are_16_byte_aligned(D, dtype, {dy, x, weight, dx}));
    if (dweight) {
      if (rows > 0)
        hipLaunchKernelGGL(rms_dw_partial_kernel<T>, cgrid, dim3(256), 0, s, static_cast<const T*>(dy),
                           static_cast<const T*>(x), rstd, static_cast<float*>(workspace), (int)rows, (int)D,
                           per);
      // no rows: the sum over nothing, zeros
      hipLaunchKernelGGL(rms_dw_final_kernel<T>, fgrid, dim3(256), 0, s, static_cast<const float*>(workspace),
                         static_cast<T*>(dweight), chunks, (int)D);
    }
  };
  if (dtype == MI355_F32) run(float{}); else run(uint16_t{});
  return check_launch("rms_norm_bwd");
}
