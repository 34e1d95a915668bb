// Grouped SwiGLU expert GEMMs in bf16 on the gfx950 matrix cores.
//
// All kernels use v_mfma_f32_32x32x16_bf16: per lane 8 bf16 of A (row lane%32,
// k = 8*(lane/32)..+7) and 8 bf16 of B (column lane%32, same k), 16 fp32 of C
// (column lane%32, rows 8*(i/4) + 4*(lane/32) + i%4).
//
// Operands reach LDS in one of two layouts, chosen by which axis is contiguous in
// HBM:
//   KC  contraction axis contiguous ([row][k], 64 k per row): 16-byte chunks are
//       XOR-swizzled by row so the 32 rows a fragment read touches hit distinct
//       banks; a fragment is one ds_read_b128.
//   KS  contraction axis strided ([k][col], col contiguous): stored as is with a
//       padded pitch; a fragment is two ds_read_b64_tr_b16, the LDS transpose read
//       that hands each lane 4 consecutive k of its own column.
// That covers every product of the block without materialising a transpose:
//   gate/up  rows . w1^T, rows . w3^T   A KC, B KC   fused SiLU*up epilogue
//   down     h . w2^T                   A KC, B KC
//   dh       dy . w2                    A KC, B KS   fused SwiGLU backward epilogue
//   drows    dgate . w1 + dup . w3      A KC, B KS   (one accumulator, K = 2F)
//   dw*      a_e^T . b_e                A KS, B KS   K = the expert's rows
//
// Row-tiled kernels take their work from the permutation plan's tile list (128
// rows of one expert each) and remap block ids so that each XCD walks a contiguous
// run of tiles: the blocks sharing an expert's weights share an L2.
#include "common.h"

namespace mi355 {
namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BM = 128, BN = 256, BK = 64;
constexpr int KS_PAD = 32;  // elements; keeps rows 16-byte aligned and shifts banks

#define LDS_PTR(p) ((__attribute__((address_space(3))) s16x4*)(p))

__device__ __forceinline__ bf16x8 frag_kc(const uint16_t* tile, int row, int kk, int lane) {
  const int r = row + (lane & 31);
  const int c = kk * 2 + (lane >> 5);
  return *reinterpret_cast<const bf16x8*>(tile + r * BK + ((c ^ (r & 7)) << 3));
}

__device__ __forceinline__ bf16x8 frag_ks(const uint16_t* tile, int col, int kk, int lane, int pitch) {
  const int g = lane >> 4, i = lane & 15;
  const uint16_t* p = tile + (kk * 16 + 8 * (g >> 1) + (i >> 2)) * pitch + col + 16 * (g & 1) + 4 * (i & 3);
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p + 4 * pitch));
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// block id -> work id such that XCD x (= bid % 8) walks ids [x*chunk, (x+1)*chunk)
__device__ __forceinline__ int xcd_remap(int bid, int total) {
  const int chunk = (total + 7) >> 3;
  const int within = bid >> 3;
  const int pid = (bid & 7) * chunk + within;
  return (within < chunk && pid < total) ? pid : -1;
}

// One 32x32 accumulator tile of the dh GEMM -> dgate / dup (bf16 rounding after dh,
// after silu(gate) and after dh*up, like the elementwise ops it replaces).
__device__ __forceinline__ void dh_epilogue_tile(const f32x16& v, const uint16_t* __restrict__ gate,
                                                 const uint16_t* __restrict__ up,
                                                 uint16_t* __restrict__ dgate,
                                                 uint16_t* __restrict__ dup, int row0, int m_base,
                                                 int valid, int f, int F) {
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int m = m_base + (i >> 2) * 8 + (i & 3);
    if (m < valid && f < F) {
      const int64_t o = static_cast<int64_t>(row0 + m) * F + f;
      const float dh = round_bf16(v[i]);
      const float g = bf16_to_f32(gate[o]);
      const float u = bf16_to_f32(up[o]);
      const float sig = 1.0f / (1.0f + __expf(-g));
      const float s = round_bf16(g * sig);
      const float ds = round_bf16(dh * u);
      dup[o] = f32_to_bf16(dh * s);
      dgate[o] = f32_to_bf16(ds * (sig * (1.0f + g * (1.0f - sig))));
    }
  }
}

enum RowMode { RM_GATEUP = 0, RM_DOWN = 1, RM_DH = 2, RM_DX = 3 };

struct RowArgs {
  const uint16_t* a0;  // GATEUP rows | DOWN h | DH dy | DX dgate
  const uint16_t* a1;  // DX dup
  const uint16_t* b0;  // GATEUP w1 | DOWN w2 | DH w2 | DX w1
  const uint16_t* b1;  // GATEUP w3 | DX w3
  uint16_t* o0;        // GATEUP gate | DOWN y | DH dgate | DX drows
  uint16_t* o1;        // GATEUP up   | DH dup
  uint16_t* o2;        // GATEUP h
  const uint16_t* gate;  // DH
  const uint16_t* up;    // DH
  const int32_t* seg_offsets;
  const int32_t* seg_counts;
  const int32_t* tile_expert;
  const int32_t* tile_row0;
  const int32_t* num_tiles;
  int D, F;
  int n_tiles;  // column tiles per row tile
};

template <int MODE>
__global__ __launch_bounds__(256, 2) void row_tiled_kernel(RowArgs p) {
  constexpr bool B_KS = (MODE == RM_DH || MODE == RM_DX);
  constexpr int B_PITCH = BN + KS_PAD;
  constexpr int B_ELEMS = B_KS ? BK * B_PITCH : BN * BK;
  __shared__ __attribute__((aligned(16))) uint16_t As[BM * BK];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[B_ELEMS];

  const int total = *p.num_tiles * p.n_tiles;
  const int pid = xcd_remap(blockIdx.x, total);
  if (pid < 0) return;
  const int tile = pid / p.n_tiles, nt = pid % p.n_tiles;
  const int e = p.tile_expert[tile];
  const int row0 = p.tile_row0[tile];
  const int valid = min(BM, p.seg_offsets[e] + p.seg_counts[e] - row0);

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = wave & 1;
  const int D = p.D, F = p.F;

  // contraction length, leading dims, output width
  const int Kdim = (MODE == RM_GATEUP || MODE == RM_DH) ? D : (MODE == RM_DOWN ? F : 2 * F);
  const int lda = (MODE == RM_GATEUP || MODE == RM_DH) ? D : F;
  const int Ncols = (MODE == RM_GATEUP || MODE == RM_DH) ? F : D;  // width of the output matrix
  const int n0 = nt * (MODE == RM_GATEUP ? BN / 2 : BN);
  const int64_t wsz = static_cast<int64_t>(D) * F;
  const uint16_t* B0 = p.b0 + e * wsz;
  const uint16_t* B1 = (MODE == RM_GATEUP || MODE == RM_DX) ? p.b1 + e * wsz : B0;
  const int64_t b1_off = B1 - B0;  // both weight stacks live in one flat address space

  // ---- global -> register staging -------------------------------------------
  // Thread `tid` moves 16-byte chunks q = tid + 256*i.  For KC tiles (8 chunks per
  // row) that is row (tid>>3) + 32*i, chunk tid&7; for KS tiles (32 chunks per k)
  // it is k = (tid>>5) + 8*i, chunk tid&31.  Only the clamped row offsets need
  // per-i storage; everything else is affine in i.
  u32x4 ra[4], rb[8];
  const int kc_row = tid >> 3, kc_chunk = tid & 7;
  const int kc_lds = kc_row * BK + ((kc_chunk ^ (kc_row & 7)) << 3);  // + i*32*BK
  const uint16_t* a_base0 = p.a0 + static_cast<int64_t>(row0) * lda + kc_chunk * 8;
  const uint16_t* a_base1 = (MODE == RM_DX) ? p.a1 + static_cast<int64_t>(row0) * lda + kc_chunk * 8 : a_base0;
  int a_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a_off[i] = min(kc_row + 32 * i, valid - 1) * lda;

  const uint16_t* b_base = B0;
  int b_off[8];
  int b_lds0, b_lds_step;
  if constexpr (!B_KS) {
    b_base += kc_chunk * 8;
    b_lds0 = kc_lds;
    b_lds_step = 32 * BK;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int r = kc_row + 32 * i;
      if constexpr (MODE == RM_GATEUP)
        b_off[i] = min(n0 + (r & 127), F - 1) * D;  // rows 0..127 from w1, 128..255 from w3
      else
        b_off[i] = min(n0 + r, D - 1) * F;  // DOWN: w2[e] is (D,F); a tile row is an output column d
    }
  } else {
    // DH: B(k=d, n=f) = w2[e][d][f], ld F.  DX: B(k=f, n=d) = w1/w3[e][f][d], ld D.
    const int ks_k = tid >> 5, ks_chunk = tid & 31;
    b_base += static_cast<int64_t>(ks_k) * Ncols + min(n0 + ks_chunk * 8, Ncols - 8);
    b_lds0 = ks_k * B_PITCH + ks_chunk * 8;
    b_lds_step = 8 * B_PITCH;
#pragma unroll
    for (int i = 0; i < 8; ++i) b_off[i] = 8 * i * Ncols;
  }

#define LOAD_REGS(K0)                                                                          \
  do {                                                                                         \
    const int k0_ = (K0);                                                                      \
    if constexpr (MODE == RM_DX) {                                                             \
      const bool second = k0_ >= F;                                                            \
      const int kk0 = second ? k0_ - F : k0_;                                                  \
      const uint16_t* ab = (second ? a_base1 : a_base0) + kk0;                                 \
      const uint16_t* bb = b_base + (second ? b1_off : 0) + static_cast<int64_t>(kk0) * Ncols; \
      _Pragma("unroll") for (int i = 0; i < 4; ++i)                                            \
          ra[i] = *reinterpret_cast<const u32x4*>(ab + a_off[i]);                              \
      _Pragma("unroll") for (int i = 0; i < 8; ++i)                                            \
          rb[i] = *reinterpret_cast<const u32x4*>(bb + b_off[i]);                              \
    } else {                                                                                   \
      const uint16_t* ab = a_base0 + k0_;                                                      \
      const uint16_t* bb = B_KS ? b_base + static_cast<int64_t>(k0_) * Ncols : b_base + k0_;   \
      _Pragma("unroll") for (int i = 0; i < 4; ++i)                                            \
          ra[i] = *reinterpret_cast<const u32x4*>(ab + a_off[i]);                              \
      _Pragma("unroll") for (int i = 0; i < 8; ++i) {                                          \
        if constexpr (MODE == RM_GATEUP)                                                       \
          rb[i] = *reinterpret_cast<const u32x4*>(bb + (i >= 4 ? b1_off : 0) + b_off[i]);      \
        else                                                                                   \
          rb[i] = *reinterpret_cast<const u32x4*>(bb + b_off[i]);                              \
      }                                                                                        \
    }                                                                                          \
  } while (0)

  f32x16 acc[2][4];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int nj = 0; nj < 4; ++nj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mi][nj][i] = 0.0f;

  // LDS row/column of this wave's four 32-wide column tiles
  int bcol[4];
#pragma unroll
  for (int nj = 0; nj < 4; ++nj) {
    if constexpr (MODE == RM_GATEUP)
      bcol[nj] = (nj < 2 ? 0 : 128) + wn * 64 + (nj & 1) * 32;
    else
      bcol[nj] = wn * 128 + nj * 32;
  }

  LOAD_REGS(0);
  for (int k0 = 0; k0 < Kdim; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(As + kc_lds + i * 32 * BK) = ra[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(Bs + b_lds0 + i * b_lds_step) = rb[i];
    __syncthreads();
    if (k0 + BK < Kdim) LOAD_REGS(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[2], bf[4];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) af[mi] = frag_kc(As, wm + mi * 32, kk, lane);
#pragma unroll
      for (int nj = 0; nj < 4; ++nj) {
        if constexpr (B_KS)
          bf[nj] = frag_ks(Bs, bcol[nj], kk, lane, B_PITCH);
        else
          bf[nj] = frag_kc(Bs, bcol[nj], kk, lane);
      }
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int nj = 0; nj < 4; ++nj)
          acc[mi][nj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bf[nj], acc[mi][nj], 0, 0, 0);
    }
    __syncthreads();
  }

  // ---- epilogue -----------------------------------------------------------------
#undef LOAD_REGS
  const int ln = lane & 31, lh = lane >> 5;
  if constexpr (MODE == RM_DH) {
    // SwiGLU backward on the accumulators: dgate = dh*up*silu'(gate), dup = dh*silu(gate)
#define DH_TILE(MI, NJ) \
  dh_epilogue_tile(acc[MI][NJ], p.gate, p.up, p.o0, p.o1, row0, wm + MI * 32 + lh * 4, valid, \
                   n0 + wn * 128 + NJ * 32 + ln, F)
    DH_TILE(0, 0); DH_TILE(0, 1); DH_TILE(0, 2); DH_TILE(0, 3);
    DH_TILE(1, 0); DH_TILE(1, 1); DH_TILE(1, 2); DH_TILE(1, 3);
#undef DH_TILE
    return;
  }
#pragma unroll
  for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = wm + mi * 32 + (i >> 2) * 8 + lh * 4 + (i & 3);
      const bool row_ok = m < valid;
      const int64_t r = row0 + m;
      if constexpr (MODE == RM_GATEUP) {
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          const int f = n0 + wn * 64 + j * 32 + ln;
          if (row_ok && f < F) {
            const uint16_t gb = f32_to_bf16(acc[mi][j][i]);
            const uint16_t ub = f32_to_bf16(acc[mi][j + 2][i]);
            const float g = bf16_to_f32(gb);
            const float s = round_bf16(g / (1.0f + __expf(-g)));
            p.o0[r * F + f] = gb;
            p.o1[r * F + f] = ub;
            p.o2[r * F + f] = f32_to_bf16(s * bf16_to_f32(ub));
          }
        }
      } else {
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) {
          const int d = n0 + wn * 128 + nj * 32 + ln;
          if (row_ok && d < D) p.o0[r * D + d] = f32_to_bf16(acc[mi][nj][i]);
        }
      }
    }
  }
}

// ---- weight gradients: C[e](M,N) = sum_{r in segment e} A[r][m] * B[r][n] ----------
struct WgradArgs {
  const uint16_t* a;  // (rows, M) row-major
  const uint16_t* b;  // (rows, N) row-major
  uint16_t* c;        // (El, M, N)
  const int32_t* seg_offsets;
  const int32_t* seg_counts;
  int M, N;
  int m_tiles, n_tiles;
  int total;  // El * m_tiles * n_tiles
};

__global__ __launch_bounds__(256, 2) void wgrad_kernel(WgradArgs p) {
  constexpr int A_PITCH = BM + KS_PAD, B_PITCH = BN + KS_PAD;
  __shared__ __attribute__((aligned(16))) uint16_t As[BK * A_PITCH];
  __shared__ __attribute__((aligned(16))) uint16_t Bs[BK * B_PITCH];

  const int per_e = p.m_tiles * p.n_tiles;
  const int pid = xcd_remap(blockIdx.x, p.total);
  if (pid < 0) return;
  const int e = pid / per_e;
  const int rem = pid % per_e;
  const int mt = rem / p.n_tiles, nt = rem % p.n_tiles;
  const int m0 = mt * BM, n0 = nt * BN;
  const int M = p.M, N = p.N;
  const int seg0 = p.seg_offsets[e], cnt = p.seg_counts[e];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;

  u32x4 ra[4], rb[8];
  int a_k[4], a_c[4], b_k[8], b_c[8];
  const uint16_t* a_ptr[4];
  const uint16_t* b_ptr[8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int q = tid + 256 * i;
    a_k[i] = q >> 4;
    a_c[i] = q & 15;
    a_ptr[i] = p.a + static_cast<int64_t>(seg0 + a_k[i]) * M + min(m0 + a_c[i] * 8, M - 8);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int q = tid + 256 * i;
    b_k[i] = q >> 5;
    b_c[i] = q & 31;
    b_ptr[i] = p.b + static_cast<int64_t>(seg0 + b_k[i]) * N + min(n0 + b_c[i] * 8, N - 8);
  }
  auto load_regs = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
      ra[i] = (k0 + a_k[i] < cnt) ? *reinterpret_cast<const u32x4*>(a_ptr[i] + static_cast<int64_t>(k0) * M)
                                  : u32x4{0, 0, 0, 0};
#pragma unroll
    for (int i = 0; i < 8; ++i)
      rb[i] = (k0 + b_k[i] < cnt) ? *reinterpret_cast<const u32x4*>(b_ptr[i] + static_cast<int64_t>(k0) * N)
                                  : u32x4{0, 0, 0, 0};
  };

  f32x16 acc[2][4];
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int nj = 0; nj < 4; ++nj)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[mi][nj][i] = 0.0f;

  if (cnt > 0) load_regs(0);
  for (int k0 = 0; k0 < cnt; k0 += BK) {
#pragma unroll
    for (int i = 0; i < 4; ++i) *reinterpret_cast<u32x4*>(As + a_k[i] * A_PITCH + a_c[i] * 8) = ra[i];
#pragma unroll
    for (int i = 0; i < 8; ++i) *reinterpret_cast<u32x4*>(Bs + b_k[i] * B_PITCH + b_c[i] * 8) = rb[i];
    __syncthreads();
    if (k0 + BK < cnt) load_regs(k0 + BK);
#pragma unroll
    for (int kk = 0; kk < BK / 16; ++kk) {
      bf16x8 af[2], bf[4];
#pragma unroll
      for (int mi = 0; mi < 2; ++mi) af[mi] = frag_ks(As, wm + mi * 32, kk, lane, A_PITCH);
#pragma unroll
      for (int nj = 0; nj < 4; ++nj) bf[nj] = frag_ks(Bs, wn + nj * 32, kk, lane, B_PITCH);
#pragma unroll
      for (int mi = 0; mi < 2; ++mi)
#pragma unroll
        for (int nj = 0; nj < 4; ++nj)
          acc[mi][nj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[mi], bf[nj], acc[mi][nj], 0, 0, 0);
    }
    __syncthreads();
  }

  uint16_t* C = p.c + static_cast<int64_t>(e) * M * N;
  const int ln = lane & 31, lh = lane >> 5;
#pragma unroll
  for (int mi = 0; mi < 2; ++mi)
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int m = m0 + wm + mi * 32 + (i >> 2) * 8 + lh * 4 + (i & 3);
      if (m >= M) continue;
#pragma unroll
      for (int nj = 0; nj < 4; ++nj) {
        const int n = n0 + wn + nj * 32 + ln;
        if (n < N) C[static_cast<int64_t>(m) * N + n] = f32_to_bf16(acc[mi][nj][i]);
      }
    }
}

}  // namespace

// ---- host side (called from grouped.hip) ---------------------------------------------
// `stages` is a mask of MI355_STAGE_* bits: which of the seven GEMM kernels to launch.
enum { STAGE_GATEUP = 1, STAGE_DOWN = 2, STAGE_DH = 4, STAGE_DX = 8, STAGE_DW2 = 16, STAGE_DW1 = 32, STAGE_DW3 = 64 };
bool bf16_fast_path_ok(int64_t D, int64_t F) { return D % 64 == 0 && F % 64 == 0 && D >= 64 && F >= 64; }

static unsigned round8(int64_t v) { return static_cast<unsigned>((v + 7) / 8 * 8); }

int bf16_grouped_fwd(const void* rows, const void* w1, const void* w3, const void* w2,
                     const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* gate, void* up, void* h, void* y, int64_t D,
                     int64_t F, int stages, hipStream_t s) {
  RowArgs a{};
  a.seg_offsets = seg_offsets; a.seg_counts = seg_counts; a.tile_expert = tile_expert;
  a.tile_row0 = tile_row0; a.num_tiles = num_tiles; a.D = (int)D; a.F = (int)F;
  a.a0 = (const uint16_t*)rows; a.b0 = (const uint16_t*)w1; a.b1 = (const uint16_t*)w3;
  a.o0 = (uint16_t*)gate; a.o1 = (uint16_t*)up; a.o2 = (uint16_t*)h;
  a.n_tiles = (int)((F + BN / 2 - 1) / (BN / 2));
  if (stages & STAGE_GATEUP) {
    hipLaunchKernelGGL(row_tiled_kernel<RM_GATEUP>, dim3(round8(tile_capacity * a.n_tiles)), dim3(256), 0, s, a);
    if (int rc = check_launch("grouped gate/up")) return rc;
  }
  if (!(stages & STAGE_DOWN)) return MI355_OK;
  RowArgs b{};
  b.seg_offsets = seg_offsets; b.seg_counts = seg_counts; b.tile_expert = tile_expert;
  b.tile_row0 = tile_row0; b.num_tiles = num_tiles; b.D = (int)D; b.F = (int)F;
  b.a0 = (const uint16_t*)h; b.b0 = (const uint16_t*)w2; b.o0 = (uint16_t*)y;
  b.n_tiles = (int)((D + BN - 1) / BN);
  hipLaunchKernelGGL(row_tiled_kernel<RM_DOWN>, dim3(round8(tile_capacity * b.n_tiles)), dim3(256), 0, s, b);
  return check_launch("grouped down");
}

int bf16_grouped_bwd(const void* dy, const void* rows, const void* w1, const void* w3,
                     const void* w2, const void* gate, const void* up, const void* h,
                     const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* dgate, void* dup, void* drows, void* dw1,
                     void* dw3, void* dw2, int64_t El, int64_t D, int64_t F, int stages,
                     hipStream_t s) {
  RowArgs a{};
  a.seg_offsets = seg_offsets; a.seg_counts = seg_counts; a.tile_expert = tile_expert;
  a.tile_row0 = tile_row0; a.num_tiles = num_tiles; a.D = (int)D; a.F = (int)F;
  a.a0 = (const uint16_t*)dy; a.b0 = (const uint16_t*)w2;
  a.gate = (const uint16_t*)gate; a.up = (const uint16_t*)up;
  a.o0 = (uint16_t*)dgate; a.o1 = (uint16_t*)dup;
  a.n_tiles = (int)((F + BN - 1) / BN);
  if (stages & STAGE_DH) {
    hipLaunchKernelGGL(row_tiled_kernel<RM_DH>, dim3(round8(tile_capacity * a.n_tiles)), dim3(256), 0, s, a);
    if (int rc = check_launch("grouped dh")) return rc;
  }
  if (drows && (stages & STAGE_DX)) {
    RowArgs b{};
    b.seg_offsets = seg_offsets; b.seg_counts = seg_counts; b.tile_expert = tile_expert;
    b.tile_row0 = tile_row0; b.num_tiles = num_tiles; b.D = (int)D; b.F = (int)F;
    b.a0 = (const uint16_t*)dgate; b.a1 = (const uint16_t*)dup;
    b.b0 = (const uint16_t*)w1; b.b1 = (const uint16_t*)w3; b.o0 = (uint16_t*)drows;
    b.n_tiles = (int)((D + BN - 1) / BN);
    hipLaunchKernelGGL(row_tiled_kernel<RM_DX>, dim3(round8(tile_capacity * b.n_tiles)), dim3(256), 0, s, b);
    if (int rc = check_launch("grouped drows")) return rc;
  }
  auto wgrad = [&](const void* A, const void* B, void* C, int64_t M, int64_t N, const char* what) {
    WgradArgs w{};
    w.a = (const uint16_t*)A; w.b = (const uint16_t*)B; w.c = (uint16_t*)C;
    w.seg_offsets = seg_offsets; w.seg_counts = seg_counts; w.M = (int)M; w.N = (int)N;
    w.m_tiles = (int)((M + BM - 1) / BM); w.n_tiles = (int)((N + BN - 1) / BN);
    w.total = (int)(El * w.m_tiles * w.n_tiles);
    hipLaunchKernelGGL(wgrad_kernel, dim3(round8(w.total)), dim3(256), 0, s, w);
    return check_launch(what);
  };
  if (dw2 && (stages & STAGE_DW2)) if (int rc = wgrad(dy, h, dw2, D, F, "grouped dw2")) return rc;
  if (dw1 && (stages & STAGE_DW1)) if (int rc = wgrad(dgate, rows, dw1, F, D, "grouped dw1")) return rc;
  if (dw3 && (stages & STAGE_DW3)) if (int rc = wgrad(dup, rows, dw3, F, D, "grouped dw3")) return rc;
  return MI355_OK;
}

}  // namespace mi355
