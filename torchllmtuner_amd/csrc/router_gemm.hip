// Router projections on the bf16 matrix cores with fp32 accuracy.
//
// The router gate is an fp32 GEMM over bf16 activations (x) and fp32 weights (W).  A
// bf16 value times a bf16 value is exact in fp32, so an fp32 operand written as the sum of
// three bf16 pieces (hi + mid + lo, 24 mantissa bits) turns the fp32 product into three
// bf16 MFMAs that accumulate in fp32 -- 16x the rate of the fp32 MFMA for 3x the
// instructions, which makes all three projections memory bound:
//   logits = x . W^T            x exact in bf16, W in three pieces
//   dW     = dlogits^T . x      dlogits in three pieces (split while it is staged)
//   dx     = dlogits . W        rounded to bf16 on output, so hi.hi + hi.mid + mid.hi
//                               (relative error 2^-16) is enough
// Shapes: D and E multiples of 64; anything else stays on the strided fp32-MFMA kernels.
#include <algorithm>
#include <cstdint>

#include "bf16_tiles.h"
#include "common.h"
#include "gemm_generic.h"

namespace mi355 {
namespace {

__device__ __forceinline__ int kc_off(int row, int chunk) {
  return row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
}
template <int COLS>
__device__ __forceinline__ int ks_off(int k, int chunk) {
  return k * COLS + ((chunk ^ ks_key(k)) << 3);
}

// 8 consecutive fp32 -> three 16-byte chunks of bf16 pieces (hi, mid, lo)
__device__ __forceinline__ void split8(const f32x4& a, const f32x4& b, u32x4& hi, u32x4& mid, u32x4& lo) {
  float v[8] = {a[0], a[1], a[2], a[3], b[0], b[1], b[2], b[3]};
  float r1[8], r2[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    r1[i] = v[i] - round_bf16(v[i]);
    r2[i] = r1[i] - round_bf16(r1[i]);
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    hi[i] = pack_bf16x2(v[2 * i], v[2 * i + 1]);
    mid[i] = pack_bf16x2(r1[2 * i], r1[2 * i + 1]);
    lo[i] = pack_bf16x2(r2[2 * i], r2[2 * i + 1]);
  }
}

// W (n fp32) -> out[s][n] bf16, s < nsplit
__global__ __launch_bounds__(256) void split_kernel(const float* __restrict__ w, uint16_t* __restrict__ out,
                                                    int64_t n, int nsplit) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 8;
  if (i >= n) return;  // n is a multiple of 8 (D % 64 == 0)
  const f32x4 a = *reinterpret_cast<const f32x4*>(w + i);
  const f32x4 b = *reinterpret_cast<const f32x4*>(w + i + 4);
  u32x4 hi, mid, lo;
  split8(a, b, hi, mid, lo);
  *reinterpret_cast<u32x4*>(out + i) = hi;
  *reinterpret_cast<u32x4*>(out + n + i) = mid;
  if (nsplit > 2) *reinterpret_cast<u32x4*>(out + 2 * n + i) = lo;
}

// ---- logits(T,E) = x(T,D) . W(E,D)^T + bias --------------------------------------------
// Tile 32 tokens x 128 experts, 4 waves each 32 x 32; per K step of 64: x tile KC (4 KiB)
// and the three weight-piece tiles KC (48 KiB); two LDS stages.
constexpr int F_BM = 32, F_BN = 128, F_NT = 256;
constexpr int F_STAGE = (F_BM + 3 * F_BN) * BK;  // elements

__global__ __launch_bounds__(F_NT) void gate_fwd_kernel(const uint16_t* __restrict__ x,
                                                        const uint16_t* __restrict__ ws,
                                                        const float* __restrict__ bias,
                                                        float* __restrict__ logits, int T, int D, int E) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int t0 = blockIdx.x * F_BM, n0 = blockIdx.y * F_BN;
  const int row = tid >> 3, chunk = tid & 7;
  const int64_t ED = static_cast<int64_t>(E) * D;
  const uint16_t* ap = x + static_cast<int64_t>(min(t0 + row, T - 1)) * D + chunk * 8;
  const uint16_t* bp[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) bp[i] = ws + static_cast<int64_t>(min(n0 + row + 32 * i, E - 1)) * D + chunk * 8;
  const int a_lds = kc_off(row, chunk);
  u32x4 ra, rb[12];
  auto fetch = [&](int k0) {
    ra = *reinterpret_cast<const u32x4*>(ap + k0);
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i) rb[s * 4 + i] = *reinterpret_cast<const u32x4*>(bp[i] + s * ED + k0);
  };
  auto park = [&](uint16_t* st) {
    *reinterpret_cast<u32x4*>(st + a_lds) = ra;
#pragma unroll
    for (int s = 0; s < 3; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
        *reinterpret_cast<u32x4*>(st + (F_BM + s * F_BN + 32 * i) * BK + a_lds) = rb[s * 4 + i];
  };
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.0f;
  const int ksteps = D / BK;
  fetch(0);
  park(smem);
  if (ksteps > 1) fetch(BK);
  __syncthreads();
  for (int ks = 0; ks < ksteps; ++ks) {
    const uint16_t* As = smem + (ks & 1) * F_STAGE;
    if (ks + 1 < ksteps) park(smem + ((ks + 1) & 1) * F_STAGE);
    if (ks + 2 < ksteps) fetch((ks + 2) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const bf16x8 af = frag_kc(As, 0, kk, lane);
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        const bf16x8 bf = frag_kc(As + (F_BM + s * F_BN) * BK, wave * 32, kk, lane);
        acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf, af, acc, 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // lane = token row (lane & 31); registers = expert columns (i>>2)*8 + (lane>>5)*4 + (i&3)
  const int t = t0 + (lane & 31);
  if (t < T) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wave * 32 + q * 8 + (lane >> 5) * 4;
      if (n < E) {  // E % 4 == 0
        f32x4 v = {acc[q * 4], acc[q * 4 + 1], acc[q * 4 + 2], acc[q * 4 + 3]};
        if (bias) v += *reinterpret_cast<const f32x4*>(bias + n);
        *reinterpret_cast<f32x4*>(logits + static_cast<int64_t>(t) * E + n) = v;
      }
    }
  }
}

// The same product for many tokens: 128 tokens x 128 experts per workgroup, 8 waves as 2 x 4
// (each 64 tokens x 32 experts), the contraction split over gridDim.z so that the grid still
// fills the chip.  The 32-token kernel above streams the three weight-piece tiles once per 32
// tokens -- at T = 8192 that is 0.4 GB through L2 for a 37 MB problem, and all of its time;
// this one streams them once per 128 tokens.  Partial sums go to the workspace and are added
// (with the bias) in split order by logits_reduce_kernel; a single split writes logits itself.
constexpr int G_BM = 128, G_BN = 128, G_NT = 512;
constexpr int G_STAGE = (G_BM + 3 * G_BN) * BK;  // elements, 64 KiB

__global__ __launch_bounds__(G_NT, 2) void gate_fwd_wide_kernel(const uint16_t* __restrict__ x,
                                                                const uint16_t* __restrict__ ws,
                                                                const float* __restrict__ bias,
                                                                float* __restrict__ out, int T, int D, int E,
                                                                int k_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 2) * 64, wn = (wave & 3) * 32;
  const int t0 = blockIdx.x * G_BM, n0 = blockIdx.y * G_BN;
  const int k_begin = blockIdx.z * k_per_split;
  const int ksteps = min(k_per_split, D - k_begin) / BK;
  const int row = tid >> 3, chunk = tid & 7;  // 64 rows per pass
  const int64_t ED = static_cast<int64_t>(E) * D;
  const uint16_t* ap[2];
  const uint16_t* bp[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    ap[i] = x + static_cast<int64_t>(min(t0 + row + 64 * i, T - 1)) * D + k_begin + chunk * 8;
    bp[i] = ws + static_cast<int64_t>(min(n0 + row + 64 * i, E - 1)) * D + k_begin + chunk * 8;
  }
  const int lds0 = kc_off(row, chunk);  // + 64 rows * BK per pass (64 % 16 == 0: same swizzle key)
  u32x4 ra[2], rb[6];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) ra[i] = *reinterpret_cast<const u32x4*>(ap[i] + k0);
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int i = 0; i < 2; ++i) rb[p * 2 + i] = *reinterpret_cast<const u32x4*>(bp[i] + p * ED + k0);
  };
  auto park = [&](uint16_t* st) {
#pragma unroll
    for (int i = 0; i < 2; ++i) *reinterpret_cast<u32x4*>(st + 64 * i * BK + lds0) = ra[i];
#pragma unroll
    for (int p = 0; p < 3; ++p)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        *reinterpret_cast<u32x4*>(st + (G_BM + p * G_BN + 64 * i) * BK + lds0) = rb[p * 2 + i];
  };
  f32x16 acc[2];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  if (ksteps > 0) {
    fetch(0);
    park(smem);
    if (ksteps > 1) fetch(BK);
  }
  __syncthreads();
  for (int ks = 0; ks < ksteps; ++ks) {
    const uint16_t* As = smem + (ks & 1) * G_STAGE;
    if (ks + 1 < ksteps) park(smem + ((ks + 1) & 1) * G_STAGE);
    if (ks + 2 < ksteps) fetch((ks + 2) * BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[2];
#pragma unroll
      for (int m = 0; m < 2; ++m) af[m] = frag_kc(As, wm + m * 32, kk, lane);
#pragma unroll
      for (int p = 0; p < 3; ++p) {
        const bf16x8 bf = frag_kc(As + (G_BM + p * G_BN) * BK, wn, kk, lane);
#pragma unroll
        for (int m = 0; m < 2; ++m) acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf, af[m], acc[m], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // lane = token row (lane & 31); registers = expert columns (i>>2)*8 + (lane>>5)*4 + (i&3)
  float* dst = out + static_cast<int64_t>(blockIdx.z) * T * E;
  const bool direct = gridDim.z == 1;
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    const int t = t0 + wm + m * 32 + (lane & 31);
    if (t >= T) continue;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const int n = n0 + wn + q * 8 + (lane >> 5) * 4;
      if (n < E) {  // E % 4 == 0
        f32x4 v = {acc[m][q * 4], acc[m][q * 4 + 1], acc[m][q * 4 + 2], acc[m][q * 4 + 3]};
        if (direct && bias) v += *reinterpret_cast<const f32x4*>(bias + n);
        *reinterpret_cast<f32x4*>(dst + static_cast<int64_t>(t) * E + n) = v;
      }
    }
  }
}

// logits[t][e] = sum over the splits, in order, of partial[z][t][e], plus bias[e]
__global__ __launch_bounds__(256) void logits_reduce_kernel(const float* __restrict__ partial,
                                                            const float* __restrict__ bias,
                                                            float* __restrict__ logits, int64_t TE, int E,
                                                            int splits) {
  const int64_t i = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) * 4;
  if (i >= TE) return;  // E % 4 == 0: a group of four never straddles a row
  f32x4 acc = *reinterpret_cast<const f32x4*>(partial + i);
  for (int z = 1; z < splits; ++z) acc += *reinterpret_cast<const f32x4*>(partial + z * TE + i);
  if (bias) acc += *reinterpret_cast<const f32x4*>(bias + i % E);
  *reinterpret_cast<f32x4*>(logits + i) = acc;
}

// ---- dx(T,D) = dlogits(T,E) . W(E,D), bf16 out ------------------------------------------
// Tile 128 tokens x 128 columns, 8 waves as 2 x 4, each 64 x 32.  Per K step of 64
// experts: dlogits tile split on the fly into hi / mid (KC), W hi / mid tiles KS.
constexpr int X_BM = 128, X_BN = 128, X_NT = 512;

__global__ __launch_bounds__(X_NT, 2) void gate_dx_kernel(const float* __restrict__ dlogits,
                                                         const uint16_t* __restrict__ ws,
                                                         uint16_t* __restrict__ dx, int T, int D, int E) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* A_hi = smem;                    // [128][64] KC
  uint16_t* A_mid = A_hi + X_BM * BK;
  uint16_t* B_hi = A_mid + X_BM * BK;       // [64][128] KS
  uint16_t* B_mid = B_hi + BK * X_BN;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 2) * 64, wn = (wave & 3) * 32;
  const int t0 = blockIdx.x * X_BM;
  const int n0 = min(static_cast<int>(blockIdx.y) * X_BN, D - X_BN);  // D >= 128: a last tile starts early
  const int64_t ED = static_cast<int64_t>(E) * D;
  f32x16 acc[2];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[m][i] = 0.0f;
  // One LDS stage; the operands of K step k+1 are requested into registers before the MFMAs of
  // step k (with nothing in flight during the MFMAs every step waited out a memory round trip).
  // A: 128 rows x 8 chunks of 8 experts = 1024 units, 2 per thread; B: 64 experts x 16 chunks =
  // 1024 units per piece, 2 per thread.
  f32x4 ra[2][2];
  u32x4 rb[2][2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int u = tid + X_NT * i;
      const float* src = dlogits + static_cast<int64_t>(min(t0 + (u >> 3), T - 1)) * E + k0 + (u & 7) * 8;
      ra[i][0] = *reinterpret_cast<const f32x4*>(src);
      ra[i][1] = *reinterpret_cast<const f32x4*>(src + 4);
      const uint16_t* bsrc = ws + static_cast<int64_t>(k0 + (u >> 4)) * D + n0 + (u & 15) * 8;
      rb[i][0] = *reinterpret_cast<const u32x4*>(bsrc);
      rb[i][1] = *reinterpret_cast<const u32x4*>(bsrc + ED);
    }
  };
  fetch(0);
  for (int k0 = 0; k0 < E; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int u = tid + X_NT * i;
      u32x4 hi, mid, lo;
      split8(ra[i][0], ra[i][1], hi, mid, lo);
      *reinterpret_cast<u32x4*>(A_hi + kc_off(u >> 3, u & 7)) = hi;
      *reinterpret_cast<u32x4*>(A_mid + kc_off(u >> 3, u & 7)) = mid;
      *reinterpret_cast<u32x4*>(B_hi + ks_off<X_BN>(u >> 4, u & 15)) = rb[i][0];
      *reinterpret_cast<u32x4*>(B_mid + ks_off<X_BN>(u >> 4, u & 15)) = rb[i][1];
    }
    __syncthreads();
    if (k0 + BK < E) fetch(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      const bf16x8 bh = frag_ks<X_BN>(B_hi, wn, kk, lane);
      const bf16x8 bm = frag_ks<X_BN>(B_mid, wn, kk, lane);
#pragma unroll
      for (int m = 0; m < 2; ++m) {
        const bf16x8 ah = frag_kc(A_hi, wm + m * 32, kk, lane);
        const bf16x8 am = frag_kc(A_mid, wm + m * 32, kk, lane);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh, ah, acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bm, ah, acc[m], 0, 0, 0);
        acc[m] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bh, am, acc[m], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // through the wave's private LDS region (64 x 32 bf16), then 16-byte row pieces
  using S = WaveStage<32>;
  uint16_t* st = smem + wave * S::ELEMS;
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int q = 0; q < 4; ++q)
      S::put4(st, m, 0, lane, q, acc[m][q * 4], acc[m][q * 4 + 1], acc[m][q * 4 + 2], acc[m][q * 4 + 3]);
  __builtin_amdgcn_s_waitcnt(0xc07f);
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int it = 0; it < 4; ++it) {
    const int idx = it * 64 + lane;
    const int m = idx >> 2, c = idx & 3;
    const int t = t0 + wm + m;
    if (t < T)
      *reinterpret_cast<u32x4*>(dx + static_cast<int64_t>(t) * D + n0 + wn + c * 8) =
          *reinterpret_cast<const u32x4*>(st + m * S::PITCH + c * 8);
  }
}

// ---- dW(E,D) = dlogits(T,E)^T . x(T,D), fp32 partials per K split -----------------------
// Tile 128 experts x 128 columns, 8 waves as 4 x 2, each 32 x 64.  Per K step of 64
// tokens: dlogits tile split into three pieces (KS), x tile (KS).
constexpr int W_BM = 128, W_BN = 128, W_NT = 512;

__global__ __launch_bounds__(W_NT, 2) void gate_dw_kernel(const float* __restrict__ dlogits,
                                                         const uint16_t* __restrict__ x,
                                                         float* __restrict__ partial, int T, int D, int E,
                                                         int rows_per_split) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* A_p = smem;                 // 3 x [64][128] KS
  uint16_t* B_s = smem + 3 * BK * W_BM;  // [64][128] KS
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 32, wn = (wave & 1) * 64;
  const int n0 = min(static_cast<int>(blockIdx.x) * W_BN, D - W_BN);
  const int m0 = blockIdx.y * W_BM;  // E % 64 == 0; a last tile of 64 experts clamps its rows
  const int split = blockIdx.z;
  const int t_begin = split * rows_per_split, t_end = min(T, t_begin + rows_per_split);
  f32x16 acc[2];
#pragma unroll
  for (int n = 0; n < 2; ++n)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[n][i] = 0.0f;
  const u32x4 zero = {0, 0, 0, 0};
  // 64 tokens x 16 chunks of 8 experts (A) / 8 columns (B) = 1024 units each, 2 per thread; one LDS
  // stage, the next K step's operands requested into registers before the MFMAs of the current one
  f32x4 ra[2][2];
  u32x4 rb[2];
  auto fetch = [&](int tk) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int u = tid + W_NT * i;
      const int k = u >> 4, c = u & 15;
      const int tc = min(tk + k, T - 1);
      const float* src = dlogits + static_cast<int64_t>(tc) * E + min(m0 + c * 8, E - 8);
      ra[i][0] = *reinterpret_cast<const f32x4*>(src);
      ra[i][1] = *reinterpret_cast<const f32x4*>(src + 4);
      rb[i] = *reinterpret_cast<const u32x4*>(x + static_cast<int64_t>(tc) * D + n0 + c * 8);
    }
  };
  if (t_begin < t_end) fetch(t_begin);
  for (int tk = t_begin; tk < t_end; tk += BK) {
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int u = tid + W_NT * i;
      const int k = u >> 4, c = u & 15;
      const bool live = tk + k < t_end;
      u32x4 hi, mid, lo;
      split8(ra[i][0], ra[i][1], hi, mid, lo);
      const int o = ks_off<W_BM>(k, c);
      *reinterpret_cast<u32x4*>(A_p + o) = live ? hi : zero;
      *reinterpret_cast<u32x4*>(A_p + BK * W_BM + o) = live ? mid : zero;
      *reinterpret_cast<u32x4*>(A_p + 2 * BK * W_BM + o) = live ? lo : zero;
      *reinterpret_cast<u32x4*>(B_s + ks_off<W_BN>(k, c)) = rb[i];
    }
    __syncthreads();
    if (tk + BK < t_end) fetch(tk + BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 bf[2];
#pragma unroll
      for (int n = 0; n < 2; ++n) bf[n] = frag_ks<W_BN>(B_s, wn + n * 32, kk, lane);
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        const bf16x8 af = frag_ks<W_BM>(A_p + s * BK * W_BM, wm, kk, lane);
#pragma unroll
        for (int n = 0; n < 2; ++n) acc[n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[n], af, acc[n], 0, 0, 0);
      }
    }
    __syncthreads();
  }
  // lane = expert row (lane & 31); registers = 4 consecutive columns
  const int e = m0 + wm + (lane & 31);
  if (e < E) {
    float* dst = partial + (static_cast<int64_t>(split) * E + e) * D + n0 + wn;
#pragma unroll
    for (int n = 0; n < 2; ++n)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const f32x4 v = {acc[n][q * 4], acc[n][q * 4 + 1], acc[n][q * 4 + 2], acc[n][q * 4 + 3]};
        *reinterpret_cast<f32x4*>(dst + n * 32 + q * 8 + (lane >> 5) * 4) = v;
      }
  }
}

template <typename K>
int set_dyn_lds(K kernel, int bytes) {
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  return e == hipSuccess ? MI355_OK : fail(MI355_ELAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
}

constexpr int F_LDS = 2 * F_STAGE * 2;                         // 106496
constexpr int G_LDS = 2 * G_STAGE * 2;                         // 131072

// Splits of the contraction for the 128-token forward kernel: enough workgroups for the chip,
// at least four K steps each, whole K steps.  0 = use the 32-token kernel (few tokens).
int fwd_splits(int64_t T, int64_t D, int64_t E) {
  if (T < 1024) return 0;
  const int64_t tiles = ((T + G_BM - 1) / G_BM) * ((E + G_BN - 1) / G_BN);
  int64_t s = 1;
  while (s < 8 && tiles * s < 256 && D % (2 * s * BK) == 0 && D / (2 * s) >= 4 * BK) s *= 2;
  return static_cast<int>(s);
}
constexpr int X_LDS = (2 * X_BM * BK + 2 * BK * X_BN) * 2;     // 65536
constexpr int W_LDS = (3 * BK * W_BM + BK * W_BN) * 2;         // 65536

// Splits of the token contraction for dW.  Two workgroups fit a CU, so the launch runs in
// rounds of 512 and its length goes as rounds x tokens per split: one more split than fills a
// round costs a whole extra round.  Each split also adds an (E, D) fp32 partial for the
// reduction to read, priced here at twelve token rows of the kernel (measured: the sum is
// within a few percent of the best split count at 8192 x 2048 x 128, 16384 x 2048 x 128 and
// 4096 x 7168 x 256).  At least four K steps per split.
int dw_splits(int64_t T, int64_t D, int64_t E) {
  const int64_t tiles = ((D + W_BN - 1) / W_BN) * ((E + W_BM - 1) / W_BM);
  const int64_t max_s = std::max<int64_t>(1, std::min<int64_t>(64, (T + 4 * BK - 1) / (4 * BK)));
  int64_t best = 1, best_cost = INT64_MAX;
  for (int64_t s = 1; s <= max_s; ++s) {
    const int64_t rows = ((T + s - 1) / s + BK - 1) / BK * BK;
    const int64_t cost = ((tiles * s + 511) / 512) * rows + 12 * s;
    if (cost < best_cost) { best = s; best_cost = cost; }
  }
  return static_cast<int>(best);
}

}  // namespace

bool router_x3_ok(int x_dtype, int w_dtype, int64_t D, int64_t E) {
  return x_dtype == MI355_BF16 && w_dtype == MI355_F32 && D % 64 == 0 && E % 64 == 0 && D >= 128;
}

int64_t router_x3_fwd_workspace(int64_t T, int64_t D, int64_t E) {
  const int s = fwd_splits(T, D, E);
  return 3 * E * D * 2 + (s > 1 ? static_cast<int64_t>(s) * T * E * 4 : 0);
}

int64_t router_x3_bwd_workspace(int64_t T, int64_t D, int64_t E) {
  return 2 * E * D * 2 + static_cast<int64_t>(dw_splits(T, D, E)) * E * D * 4;
}

int router_x3_fwd(const void* x, const float* w, const float* bias, float* logits, void* workspace, int64_t T,
                  int64_t D, int64_t E, hipStream_t s) {
  static PerDeviceOnce configured;
  if (configured.needed()) {
    if (int rc = set_dyn_lds(gate_fwd_kernel, F_LDS)) return rc;
    configured.done();
  }
  uint16_t* ws = static_cast<uint16_t*>(workspace);
  const int64_t n = E * D;
  hipLaunchKernelGGL(split_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s, w, ws, n, 3);
  if (const int splits = fwd_splits(T, D, E)) {
    static PerDeviceOnce wide_configured;
    if (wide_configured.needed()) {
      if (int rc = set_dyn_lds(gate_fwd_wide_kernel, G_LDS)) return rc;
      wide_configured.done();
    }
    float* partial = reinterpret_cast<float*>(ws + 3 * n);  // behind the weight pieces
    const dim3 grid((unsigned)((T + G_BM - 1) / G_BM), (unsigned)((E + G_BN - 1) / G_BN), (unsigned)splits);
    hipLaunchKernelGGL(gate_fwd_wide_kernel, grid, dim3(G_NT), G_LDS, s, static_cast<const uint16_t*>(x), ws, bias,
                       splits > 1 ? partial : logits, (int)T, (int)D, (int)E, (int)(D / splits));
    if (splits > 1) {
      const int64_t te = T * E;
      hipLaunchKernelGGL(logits_reduce_kernel, dim3((unsigned)((te / 4 + 255) / 256)), dim3(256), 0, s, partial, bias,
                         logits, te, (int)E, splits);
    }
    return check_launch("router_gate_fwd");
  }
  hipLaunchKernelGGL(gate_fwd_kernel, dim3((unsigned)((T + F_BM - 1) / F_BM), (unsigned)((E + F_BN - 1) / F_BN)),
                     dim3(F_NT), F_LDS, s, static_cast<const uint16_t*>(x), ws, bias, logits, (int)T, (int)D, (int)E);
  return check_launch("router_gate_fwd");
}

int router_x3_bwd(const float* dlogits, const void* x, const float* w, void* dx, float* dw, void* workspace,
                  int64_t T, int64_t D, int64_t E, hipStream_t s) {
  static PerDeviceOnce configured;
  if (configured.needed()) {
    if (int rc = set_dyn_lds(gate_dx_kernel, X_LDS)) return rc;
    if (int rc = set_dyn_lds(gate_dw_kernel, W_LDS)) return rc;
    configured.done();
  }
  uint16_t* ws = static_cast<uint16_t*>(workspace);
  const int64_t n = E * D;
  if (dx && T > 0) {
    hipLaunchKernelGGL(split_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, s, w, ws, n, 2);
    hipLaunchKernelGGL(gate_dx_kernel, dim3((unsigned)((T + X_BM - 1) / X_BM), (unsigned)((D + X_BN - 1) / X_BN)),
                       dim3(X_NT), X_LDS, s, dlogits, ws, static_cast<uint16_t*>(dx), (int)T, (int)D, (int)E);
    if (int rc = check_launch("router_gate_bwd dx")) return rc;
  }
  if (dw) {
    const int splits = dw_splits(T, D, E);
    const int rows_per_split = (int)(((T + splits - 1) / splits + BK - 1) / BK * BK);
    float* partial = reinterpret_cast<float*>(ws + 2 * n);
    hipLaunchKernelGGL(gate_dw_kernel,
                       dim3((unsigned)((D + W_BN - 1) / W_BN), (unsigned)((E + W_BM - 1) / W_BM), (unsigned)splits),
                       dim3(W_NT), W_LDS, s, dlogits, static_cast<const uint16_t*>(x), partial, (int)T, (int)D,
                       (int)E, rows_per_split);
    if (int rc = check_launch("router_gate_bwd dw")) return rc;
    return launch_splitk_reduce(partial, dw, MI355_F32, n, splits, s);
  }
  return MI355_OK;
}

}  // namespace mi355
