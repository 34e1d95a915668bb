// Generic strided GEMM on the fp32 matrix cores (see gemm_generic.h).
//
// Workgroup = 256 lanes = 4 waves, output tile 64x64, each wave owns one 32x32
// quadrant as a single v_mfma_f32_32x32x2_f32 accumulator (16 VGPRs).  K is
// consumed in slabs of 16 staged through LDS as As[k][m] / Bs[k][n], so the
// per-lane operand of the MFMA (one A(m,k), one B(k,n)) is a conflict-free
// ds_read_b32 whatever the global layout was.  Global loads pick the lane mapping
// that walks the operand's contiguous axis.
//
// fp64 storage: an fp64 operand or result next to fp32 ones is converted on the way in and
// out (the router, which computes in fp32 whatever it is given).  With A, B and C all fp64
// (fp64 experts) the same kernel computes in fp64: each wave's 32x32 quadrant is then 2 x 2
// tiles of v_mfma_f64_16x16x4_f64.
#include "gemm_generic.h"

#include <cstdint>
#include <type_traits>

namespace mi355 {

namespace {

typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef double f64x4 __attribute__((ext_vector_type(4)));

// the arithmetic type of a product: fp64 only when everything is fp64
template <typename TA, typename TB, typename TC>
struct ComputeOf { using type = float; };
template <>
struct ComputeOf<double, double, double> { using type = double; };

template <typename CT, typename T>
__device__ __forceinline__ CT load_op(const T* p) {
  if constexpr (std::is_same_v<CT, double>) return *p;  // (T is double here)
  else return load_as_f32(p);
}
template <typename CT, typename T>
__device__ __forceinline__ void store_op(T* p, CT v) {
  if constexpr (std::is_same_v<CT, double>) *p = v;
  else store_from_f32(p, v);
}

constexpr int TM = 64, TN = 64, TK = 16, PITCH = 65;

template <typename TA, typename TB, typename TC>
__global__ __launch_bounds__(256) void ggemm_kernel(GemmArgs g) {
  using CT = typename ComputeOf<TA, TB, TC>::type;
  constexpr bool F64 = std::is_same_v<CT, double>;
  __shared__ CT As[TK][PITCH];
  __shared__ CT Bs[TK][PITCH];

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = tid >> 6;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;

  const TA* A = static_cast<const TA*>(g.A);
  const TB* B = static_cast<const TB*>(g.B);
  TC* C = static_cast<TC*>(g.C);

  int m0, n0 = blockIdx.y * TN;
  int m_valid;          // rows of this tile that exist
  int64_t row_base = 0; // ROWSEG: first global row of the tile
  int k_begin = 0, k_end = g.K;
  float* Cpartial = nullptr;

  if (g.mode == GEMM_ROWSEG) {
    const int subs = g.tile_m / TM;
    const int tile = blockIdx.x / subs, sub = blockIdx.x % subs;
    if (tile >= *g.num_tiles) return;
    const int e = g.tile_expert[tile];
    const int r0 = g.tile_row0[tile] + sub * TM;
    // the tile's rows end with its (equalised) height or with the segment
    const int cnt = g.seg_counts[e];
    const int tile_end = min(g.tile_row0[tile] + even_tile_rows(cnt, g.tile_m), g.seg_offsets[e] + cnt);
    m_valid = min(TM, tile_end - r0);
    if (m_valid <= 0) return;
    row_base = r0;
    m0 = 0;
    B += static_cast<int64_t>(e) * g.b_es;
  } else if (g.mode == GEMM_KSEG) {
    const int e = blockIdx.z;
    m0 = blockIdx.x * TM;
    m_valid = min(TM, g.M - m0);
    k_begin = g.seg_offsets[e];
    k_end = k_begin + g.seg_counts[e];
    C += static_cast<int64_t>(e) * g.c_es;
  } else {
    m0 = blockIdx.x * TM;
    m_valid = min(TM, g.M - m0);
    if (g.ksplit > 1) {
      const int chunk = ((g.K + g.ksplit - 1) / g.ksplit + TK - 1) / TK * TK;
      k_begin = blockIdx.z * chunk;
      k_end = min(g.K, k_begin + chunk);
      Cpartial = reinterpret_cast<float*>(g.C) + static_cast<int64_t>(blockIdx.z) * g.M * g.ldc;
    }
  }
  const int n_valid = min(TN, g.N - n0);
  const int64_t a_row0 = row_base + m0;

  // lane mappings for the global->LDS copy: walk the contiguous axis with lanes
  const bool a_kc = (g.a_cs == 1);
  const bool b_nc = (g.b_cs == 1);
  int am[4], ak[4], bk[4], bn[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int i = tid + j * 256;
    if (a_kc) { ak[j] = i % TK; am[j] = i / TK; } else { am[j] = i % TM; ak[j] = i / TM; }
    if (b_nc) { bn[j] = i % TN; bk[j] = i / TN; } else { bk[j] = i % TK; bn[j] = i / TK; }
  }

  CT ra[4], rb[4];
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int k = k0 + ak[j];
      ra[j] = (am[j] < m_valid && k < k_end)
                  ? load_op<CT>(A + (a_row0 + am[j]) * g.a_rs + static_cast<int64_t>(k) * g.a_cs)
                  : CT(0);
      const int kb = k0 + bk[j];
      rb[j] = (bn[j] < n_valid && kb < k_end)
                  ? load_op<CT>(B + static_cast<int64_t>(kb) * g.b_rs + static_cast<int64_t>(n0 + bn[j]) * g.b_cs)
                  : CT(0);
    }
  };

  f32x16 acc;       // fp32: one 32x32 tile
  f64x4 acc64[2][2];  // fp64: 2 x 2 tiles of 16x16
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc64[i][j][v] = 0.0;

  if (k_begin < k_end) load_slab(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += TK) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      As[ak[j]][am[j]] = ra[j];
      Bs[bk[j]][bn[j]] = rb[j];
    }
    __syncthreads();
    if (k0 + TK < k_end) load_slab(k0 + TK);
    if constexpr (F64) {
      // lane l supplies A(m = l % 16, k = l / 16) and B(k = l / 16, n = l % 16) of a 16x16x4 step
#pragma unroll
      for (int kk = 0; kk < TK; kk += 4) {
        double a[2], b[2];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          a[i] = As[kk + (lane >> 4)][wm + 16 * i + (lane & 15)];
          b[i] = Bs[kk + (lane >> 4)][wn + 16 * i + (lane & 15)];
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc64[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(a[i], b[j], acc64[i][j], 0, 0, 0);
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < TK; kk += 2) {
        const float a = As[kk + (lane >> 5)][wm + (lane & 31)];
        const float b = Bs[kk + (lane >> 5)][wn + (lane & 31)];
        acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
      }
    }
    __syncthreads();
  }

  if constexpr (F64) {
    // register v of tile (i, j) holds row 16 i + 4 v + l / 16, column 16 j + l % 16 (probed on the card)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int n = wn + 16 * j + (lane & 15);
        if (n >= n_valid) continue;
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const int m = wm + 16 * i + 4 * v + (lane >> 4);
          if (m >= m_valid) continue;
          const int64_t off = (a_row0 + m) * g.ldc + n0 + n;
          double r = acc64[i][j][v];
          if (g.accumulate) r += load_op<CT>(C + off);
          store_op<CT>(C + off, r);
        }
      }
    return;
  }

  const int n = wn + (lane & 31);
  if (n >= n_valid) return;
  const float bias = g.bias ? g.bias[n0 + n] : 0.0f;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int m = wm + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
    if (m >= m_valid) continue;
    const int64_t off = (a_row0 + m) * g.ldc + n0 + n;
    if (Cpartial) {
      Cpartial[off] = acc[i];
    } else {
      float v = acc[i] + bias;
      if (g.accumulate) v += load_as_f32(C + off);
      store_from_f32(C + off, v);
    }
  }
}

// ---- dense GEMM with 16-byte (fp32) / 8-byte (bf16) vector loads -------------------------
// Same 64x64 tile and fp32 MFMA as above, 32-deep K slabs, for the DENSE mode when the
// operands allow 4-element vector loads along their contiguous axis (the router
// projections).  AV / BV: 0 = the K axis is contiguous, 1 = the M (resp. N) axis is.
constexpr int VK = 32, VPITCH = 68;

template <typename T>
__device__ __forceinline__ void load4(const T* p, float (&v)[4]);
template <>
__device__ __forceinline__ void load4<float>(const float* p, float (&v)[4]) {
  const float4 t = *reinterpret_cast<const float4*>(p);
  v[0] = t.x; v[1] = t.y; v[2] = t.z; v[3] = t.w;
}
template <>
__device__ __forceinline__ void load4<uint16_t>(const uint16_t* p, float (&v)[4]) {
  const uint2 t = *reinterpret_cast<const uint2*>(p);
  v[0] = __uint_as_float(t.x << 16); v[1] = __uint_as_float(t.x & 0xffff0000u);
  v[2] = __uint_as_float(t.y << 16); v[3] = __uint_as_float(t.y & 0xffff0000u);
}

template <typename TA, typename TB, typename TC, int AV, int BV>
__global__ __launch_bounds__(256) void dense_vec_kernel(GemmArgs g) {
  __shared__ __attribute__((aligned(16))) float As[VK][VPITCH];
  __shared__ __attribute__((aligned(16))) float Bs[VK][VPITCH];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 32;
  const TA* A = static_cast<const TA*>(g.A);
  const TB* B = static_cast<const TB*>(g.B);
  const int m0 = blockIdx.x * TM, n0 = blockIdx.y * TN;
  int k_begin = 0, k_end = g.K;
  float* Cpartial = nullptr;
  if (g.ksplit > 1) {
    const int chunk = ((g.K + g.ksplit - 1) / g.ksplit + VK - 1) / VK * VK;
    k_begin = blockIdx.z * chunk;
    k_end = min(g.K, k_begin + chunk);
    Cpartial = reinterpret_cast<float*>(g.C) + static_cast<int64_t>(blockIdx.z) * g.M * g.ldc;
  }
  // two 4-vectors of A and two of B per thread and slab
  int am[2], ak[2], bk[2], bn[2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int i = tid + j * 256;
    if (AV == 0) { ak[j] = (i & 7) * 4; am[j] = i >> 3; } else { am[j] = (i & 15) * 4; ak[j] = i >> 4; }
    if (BV == 0) { bk[j] = (i & 7) * 4; bn[j] = i >> 3; } else { bn[j] = (i & 15) * 4; bk[j] = i >> 4; }
  }
  float ra[2][4], rb[2][4];
  auto load_slab = [&](int k0) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const bool a_ok = (m0 + am[j] < g.M) && (k0 + ak[j] < k_end);
      if (a_ok) load4<TA>(A + static_cast<int64_t>(m0 + am[j]) * g.a_rs + static_cast<int64_t>(k0 + ak[j]) * g.a_cs, ra[j]);
      else ra[j][0] = ra[j][1] = ra[j][2] = ra[j][3] = 0.0f;
      const bool b_ok = (n0 + bn[j] < g.N) && (k0 + bk[j] < k_end);
      if (b_ok) load4<TB>(B + static_cast<int64_t>(k0 + bk[j]) * g.b_rs + static_cast<int64_t>(n0 + bn[j]) * g.b_cs, rb[j]);
      else rb[j][0] = rb[j][1] = rb[j][2] = rb[j][3] = 0.0f;
    }
  };
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  if (k_begin < k_end) load_slab(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += VK) {
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      if (AV == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) As[ak[j] + q][am[j]] = ra[j][q];
      } else {
        *reinterpret_cast<float4*>(&As[ak[j]][am[j]]) = make_float4(ra[j][0], ra[j][1], ra[j][2], ra[j][3]);
      }
      if (BV == 0) {
#pragma unroll
        for (int q = 0; q < 4; ++q) Bs[bk[j] + q][bn[j]] = rb[j][q];
      } else {
        *reinterpret_cast<float4*>(&Bs[bk[j]][bn[j]]) = make_float4(rb[j][0], rb[j][1], rb[j][2], rb[j][3]);
      }
    }
    __syncthreads();
    if (k0 + VK < k_end) load_slab(k0 + VK);
#pragma unroll
    for (int kk = 0; kk < VK; kk += 2) {
      const float a = As[kk + (lane >> 5)][wm + (lane & 31)];
      const float b = Bs[kk + (lane >> 5)][wn + (lane & 31)];
      acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc, 0, 0, 0);
    }
    __syncthreads();
  }
  const int n = n0 + wn + (lane & 31);
  if (n >= g.N) return;
  const float bias = g.bias ? g.bias[n] : 0.0f;
  TC* C = static_cast<TC*>(g.C);
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int m = m0 + wm + (i >> 2) * 8 + (lane >> 5) * 4 + (i & 3);
    if (m >= g.M) continue;
    const int64_t off = static_cast<int64_t>(m) * g.ldc + n;
    if (Cpartial) Cpartial[off] = acc[i];
    else store_from_f32(C + off, acc[i] + bias);
  }
}

template <typename TC>
__global__ void splitk_reduce_kernel(const float* __restrict__ partial, TC* __restrict__ out,
                                     int64_t MN, int ksplit) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= MN) return;
  float s = 0.0f;
  for (int z = 0; z < ksplit; ++z) s += partial[z * MN + i];
  store_from_f32(out + i, s);
}

template <typename TA, typename TB>
int launch_c(const GemmArgs& a, int c_dtype, dim3 grid, hipStream_t s) {
  if (c_dtype == MI355_F32 || a.ksplit > 1)
    hipLaunchKernelGGL((ggemm_kernel<TA, TB, float>), grid, dim3(256), 0, s, a);
  else if (c_dtype == MI355_F64)
    hipLaunchKernelGGL((ggemm_kernel<TA, TB, double>), grid, dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL((ggemm_kernel<TA, TB, uint16_t>), grid, dim3(256), 0, s, a);
  return check_launch("ggemm");
}

template <typename TA>
int launch_b(const GemmArgs& a, int b_dtype, int c_dtype, dim3 grid, hipStream_t s) {
  if (b_dtype == MI355_F32) return launch_c<TA, float>(a, c_dtype, grid, s);
  if (b_dtype == MI355_BF16) return launch_c<TA, uint16_t>(a, c_dtype, grid, s);
  return launch_c<TA, double>(a, c_dtype, grid, s);
}

}  // namespace

namespace {

template <typename TA, typename TB, int AV, int BV>
int launch_vec(const GemmArgs& a, int c_dtype, dim3 grid, hipStream_t s) {
  if (c_dtype == MI355_F32 || a.ksplit > 1)
    hipLaunchKernelGGL((dense_vec_kernel<TA, TB, float, AV, BV>), grid, dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL((dense_vec_kernel<TA, TB, uint16_t, AV, BV>), grid, dim3(256), 0, s, a);
  return check_launch("dense_vec_gemm");
}

template <typename TA, typename TB>
int launch_vec_layout(const GemmArgs& a, int av, int bv, int c_dtype, dim3 grid, hipStream_t s) {
  if (av == 0 && bv == 0) return launch_vec<TA, TB, 0, 0>(a, c_dtype, grid, s);
  if (av == 0 && bv == 1) return launch_vec<TA, TB, 0, 1>(a, c_dtype, grid, s);
  if (av == 1 && bv == 0) return launch_vec<TA, TB, 1, 0>(a, c_dtype, grid, s);
  return launch_vec<TA, TB, 1, 1>(a, c_dtype, grid, s);
}

// The vector kernel applies to a dense, non-accumulating problem whose operands are
// 4-element aligned along a unit-stride axis.
bool vec_layout(const GemmArgs& a, int a_dtype, int b_dtype, int* av, int* bv) {
  if (a.mode != GEMM_DENSE || a.accumulate) return false;
  if (a_dtype == MI355_F64 || b_dtype == MI355_F64) return false;
  const int64_t asz = a_dtype == MI355_F32 ? 4 : 2, bsz = b_dtype == MI355_F32 ? 4 : 2;
  if (reinterpret_cast<uintptr_t>(a.A) % (4 * asz) || reinterpret_cast<uintptr_t>(a.B) % (4 * bsz)) return false;
  if (a.K % 4) return false;
  if (a.a_cs == 1 && a.a_rs % 4 == 0) *av = 0;
  else if (a.a_rs == 1 && a.a_cs % 4 == 0 && a.M % 4 == 0) *av = 1;
  else return false;
  if (a.b_rs == 1 && a.b_cs % 4 == 0) *bv = 0;
  else if (a.b_cs == 1 && a.b_rs % 4 == 0 && a.N % 4 == 0) *bv = 1;
  else return false;
  if (a.ksplit > 1) {
    const int chunk = ((a.K + a.ksplit - 1) / a.ksplit + VK - 1) / VK * VK;
    if (chunk % 4) return false;
  }
  return true;
}

}  // namespace

int launch_gemm(const GemmArgs& a, int a_dtype, int b_dtype, int c_dtype, dim3 grid,
                hipStream_t s) {
  if (grid.x == 0 || grid.y == 0 || grid.z == 0) return MI355_OK;
  int av = 0, bv = 0;
  if (c_dtype != MI355_F64 && vec_layout(a, a_dtype, b_dtype, &av, &bv)) {
    if (a_dtype == MI355_F32 && b_dtype == MI355_F32) return launch_vec_layout<float, float>(a, av, bv, c_dtype, grid, s);
    if (a_dtype == MI355_BF16 && b_dtype == MI355_F32) return launch_vec_layout<uint16_t, float>(a, av, bv, c_dtype, grid, s);
    if (a_dtype == MI355_F32 && b_dtype == MI355_BF16) return launch_vec_layout<float, uint16_t>(a, av, bv, c_dtype, grid, s);
    if (a_dtype == MI355_BF16 && b_dtype == MI355_BF16) return launch_vec_layout<uint16_t, uint16_t>(a, av, bv, c_dtype, grid, s);
  }
  auto known = [](int d) { return d == MI355_F32 || d == MI355_BF16 || d == MI355_F64; };
  if (!known(a_dtype) || !known(b_dtype) || !known(c_dtype))
    return fail(MI355_EINVAL, "gemm: unknown dtype %d/%d/%d", a_dtype, b_dtype, c_dtype);
  if (a.ksplit > 1 && a_dtype == MI355_F64 && b_dtype == MI355_F64 && c_dtype == MI355_F64)
    return fail(MI355_EUNSUP, "gemm: fp64 products are not split along K");
  if (a_dtype == MI355_F32) return launch_b<float>(a, b_dtype, c_dtype, grid, s);
  if (a_dtype == MI355_BF16) return launch_b<uint16_t>(a, b_dtype, c_dtype, grid, s);
  return launch_b<double>(a, b_dtype, c_dtype, grid, s);
}

dim3 gemm_grid_dense(int M, int N, int ksplit) {
  return dim3((M + TM - 1) / TM, (N + TN - 1) / TN, ksplit > 1 ? ksplit : 1);
}
dim3 gemm_grid_rowseg(int64_t tile_capacity, int tile_m, int N) {
  return dim3(static_cast<unsigned>(tile_capacity * (tile_m / TM)), (N + TN - 1) / TN, 1);
}
dim3 gemm_grid_kseg(int M, int N, int El) {
  return dim3((M + TM - 1) / TM, (N + TN - 1) / TN, El);
}

int launch_splitk_reduce(const float* partial, void* out, int out_dtype, int64_t MN, int ksplit,
                         hipStream_t s) {
  if (MN == 0) return MI355_OK;
  const unsigned blocks = static_cast<unsigned>((MN + 255) / 256);
  if (out_dtype == MI355_F32)
    hipLaunchKernelGGL(splitk_reduce_kernel<float>, dim3(blocks), dim3(256), 0, s, partial,
                       static_cast<float*>(out), MN, ksplit);
  else if (out_dtype == MI355_F64)
    hipLaunchKernelGGL(splitk_reduce_kernel<double>, dim3(blocks), dim3(256), 0, s, partial,
                       static_cast<double*>(out), MN, ksplit);
  else
    hipLaunchKernelGGL(splitk_reduce_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s, partial,
                       static_cast<uint16_t*>(out), MN, ksplit);
  return check_launch("splitk_reduce");
}

}  // namespace mi355
