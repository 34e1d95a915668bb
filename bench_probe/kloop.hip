// Stand-alone K loops of the grouped GEMMs' shape, used by the benchmark only (not part of the
// MoE C ABI): 256 x 256 x 64 tile steps over operands of the caller's choice, no tile list, no
// epilogue, every tile full.  They answer three questions the product kernels cannot be asked
// directly: what a change of the loop's schedule is worth with every operand resident on the
// chip, what is left of that once half of each step's operands stream from HBM the way an
// expert's weights do, and how the loop's energy divides between the MFMAs, the fragment reads
// from LDS and the staging of the next step's operands into LDS.  Variants:
//   0  the product's loop: per K32 block the A fragments, then two halves of four B fragments,
//      a quarter of the next step's staging (global -> registers -> LDS) with each half, and the
//      MFMAs of each 16-row block behind a wave-uniform branch (the skip of empty blocks);
//   1  the same without the branches;
//   2  operands loaded straight into LDS (buffer loads with the LDS destination; the swizzle of
//      the layout is applied on the global side), requested one K step ahead;
//   3  four waves, 128 x 128 per wave (a third fewer fragment reads), fragments of the next K32
//      block read before the MFMAs of the current one;
//   4  variant 1 with the staging but without the fragment reads (the MFMAs reuse the fragments
//      of the first step);
//   5  variant 1 with the fragment reads but without the staging (LDS keeps its first contents);
//   6  variant 1 with neither: the MFMAs alone.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

constexpr int BK = 64, BM = 256, BN = 256, STAGE = (BM + BN) * BK;  // elements per LDS stage
constexpr int kRing = 32;          // K steps after which the resident operands repeat
constexpr int kStreamSteps = 512;  // K steps after which the streamed operands repeat
constexpr long kStreamStep = 16384;  // elements streamed per K step and workgroup (32 KB)

// fragment of v_mfma_f32_16x16x32_bf16 from a [row][64 k] tile, 16-byte chunks swizzled by (row >> 1) & 7
__device__ __forceinline__ bf16x8 frag16(const uint16_t* tile, int row, int kk32, int lane) {
  const int r = row + (lane & 15);
  const int c = kk32 * 4 + (lane >> 4);
  return *reinterpret_cast<const bf16x8*>(tile + r * BK + ((c ^ ((r >> 1) & 7)) << 3));
}

// the first two stages hold some operand values before the first loads land
__device__ __forceinline__ void seed_lds(uint16_t* smem, const uint16_t* g, int tid, int nt) {
  for (int i = tid; i < 2 * STAGE; i += nt) smem[i] = g[i];
}

__device__ __forceinline__ void load_to_lds(u32x4 rs, uint32_t dst, uint32_t voffset, int soffset) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
               :
               : "s"(dst), "v"(voffset), "s"(rs), "s"(soffset)
               : "memory", "m0");
}
__device__ __forceinline__ u32x4 buffer_words(const void* base) {
  const uint64_t b = reinterpret_cast<uint64_t>(base);
  u32x4 r;
  r[0] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b));
  r[1] = __builtin_amdgcn_readfirstlane(static_cast<uint32_t>(b >> 32) & 0xffffu);
  r[2] = 0xffffffffu;
  r[3] = 0x00020000u;
  return r;
}

// resident operands: workgroup b reads a window of (BM + BN) rows x 2048 k starting at element
// b * hot_stride of `hot`; streamed operands (STREAM): the B half of a step instead comes from
// `cold`, 32 KB per step and workgroup that no other step or workgroup touches
template <int BRANCHES, int STREAM, int FRAGMENTS = 1, int STAGING = 1>
__global__ __launch_bounds__(512) void kloop_product(const uint16_t* __restrict__ hot, const uint16_t* __restrict__ cold,
                                                     float* out, int ksteps, long hot_stride, int active) {
  constexpr int NT = 512;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;
  seed_lds(smem, hot, tid, NT);
  __syncthreads();
  f32x4 acc[4][8];
  for (int a = 0; a < 4; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) acc[a][b][i] = 0.f;
  u32x4 st[8];
  const int row = tid >> 3, chunk = tid & 7;
  const int lds0 = row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
  const uint16_t* gp = hot + static_cast<long>(blockIdx.x) * hot_stride + row * 2048 + chunk * 8;
  for (int i = 0; i < 8; ++i) st[i] = *reinterpret_cast<const u32x4*>(gp + static_cast<long>(i) * (NT / 8) * 2048);
  const int act = __builtin_amdgcn_readfirstlane(active);
  bf16x8 af0[4], bf0[8];  // the first step's fragments, all the MFMAs see without FRAGMENTS
  for (int a = 0; a < 4; ++a) af0[a] = frag16(smem, wm + a * 16, 0, lane);
  for (int b = 0; b < 8; ++b) bf0[b] = frag16(smem + BM * BK, wn + b * 16, 0, lane);
  for (int ks = 0; ks < ksteps; ++ks) {
    const uint16_t* As = smem + (ks & 1) * STAGE;
    const uint16_t* Bs = As + BM * BK;
    uint16_t* Nx = smem + ((ks + 1) & 1) * STAGE;
    const uint16_t* gk = gp + ((ks + 2) % kRing) * 64;
    const uint16_t* gb = cold + (static_cast<long>(blockIdx.x) * kStreamSteps + ((ks + 2) % kStreamSteps)) * kStreamStep +
                         row * 64 + chunk * 8;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      bf16x8 af[4];
#pragma unroll
      for (int a = 0; a < 4; ++a) af[a] = FRAGMENTS ? frag16(As, wm + a * 16, kk, lane) : af0[a];
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) {
        bf16x8 bf[4];
#pragma unroll
        for (int b = 0; b < 4; ++b) bf[b] = FRAGMENTS ? frag16(Bs, wn + (hb * 4 + b) * 16, kk, lane) : bf0[hb * 4 + b];
        const int q = kk * 2 + hb;
#pragma unroll
        for (int i = q * 2; STAGING && i < q * 2 + 2; ++i) {
          *reinterpret_cast<u32x4*>(Nx + lds0 + i * (NT / 8) * BK) = st[i];
          st[i] = (STREAM && i >= 4) ? *reinterpret_cast<const u32x4*>(gb + (i - 4) * 4096)
                                     : *reinterpret_cast<const u32x4*>(gk + static_cast<long>(i) * (NT / 8) * 2048);
        }
#pragma unroll
        for (int a = 0; a < 4; ++a) {
          if (!BRANCHES || a < act) {
#pragma unroll
            for (int b = 0; b < 4; ++b)
              acc[a][hb * 4 + b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[b], af[a], acc[a][hb * 4 + b], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  }
  float s = 0.f;
  for (int a = 0; a < 4; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) s += acc[a][b][i];
  if (s == 12345.f) out[0] = s;  // keeps the loop alive
}

template <int STREAM>
__global__ __launch_bounds__(512) void kloop_direct(const uint16_t* __restrict__ hot, const uint16_t* __restrict__ cold,
                                                    float* out, int ksteps, long hot_stride) {
  constexpr int NT = 512;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;
  seed_lds(smem, hot, tid, NT);
  __syncthreads();
  f32x4 acc[4][8];
  for (int a = 0; a < 4; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) acc[a][b][i] = 0.f;
  // the lane whose piece lands in chunk position c of its row fetches the chunk that belongs there
  const int row = tid >> 3, chunk = (tid & 7) ^ ((row >> 1) & 7);
  const u32x4 rs = buffer_words(hot + static_cast<long>(blockIdx.x) * hot_stride);
  const uint32_t voff = (row * 2048 + chunk * 8) * 2, voffb = (row * 64 + chunk * 8) * 2;
  for (int ks = 0; ks < ksteps; ++ks) {
    const uint16_t* As = smem + (ks & 1) * STAGE;
    const uint16_t* Bs = As + BM * BK;
    const uint32_t nx = ((ks + 1) & 1) * STAGE * 2;
    const int koff = ((ks + 1) % kRing) * 64 * 2;
    const u32x4 rsb = buffer_words(cold + (static_cast<long>(blockIdx.x) * kStreamSteps + ((ks + 1) % kStreamSteps)) * kStreamStep);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (STREAM && i >= 4)
        load_to_lds(rsb, nx + (i * (NT / 8) + wave * 8) * 128, voffb, (i - 4) * 4096 * 2);
      else
        load_to_lds(rs, nx + (i * (NT / 8) + wave * 8) * 128, voff, koff + i * (NT / 8) * 2048 * 2);
    }
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      bf16x8 af[4], bf[8];
#pragma unroll
      for (int a = 0; a < 4; ++a) af[a] = frag16(As, wm + a * 16, kk, lane);
#pragma unroll
      for (int b = 0; b < 8; ++b) bf[b] = frag16(Bs, wn + b * 16, kk, lane);
#pragma unroll
      for (int a = 0; a < 4; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[b], af[a], acc[a][b], 0, 0, 0);
    }
    // everything this wave requested has landed in LDS, then the workgroup meets
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");
  }
  float s = 0.f;
  for (int a = 0; a < 4; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) s += acc[a][b][i];
  if (s == 12345.f) out[0] = s;
}

template <int STREAM>
__global__ __launch_bounds__(256) void kloop_four_waves(const uint16_t* __restrict__ hot, const uint16_t* __restrict__ cold,
                                                        float* out, int ksteps, long hot_stride) {
  constexpr int NT = 256;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 128, wn = (wave & 1) * 128;
  seed_lds(smem, hot, tid, NT);
  __syncthreads();
  f32x4 acc[8][8];
  for (int a = 0; a < 8; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) acc[a][b][i] = 0.f;
  u32x4 st[16];
  const int row = tid >> 3, chunk = tid & 7;
  const int lds0 = row * BK + ((chunk ^ ((row >> 1) & 7)) << 3);
  const uint16_t* gp = hot + static_cast<long>(blockIdx.x) * hot_stride + row * 2048 + chunk * 8;
  for (int i = 0; i < 16; ++i) st[i] = *reinterpret_cast<const u32x4*>(gp + static_cast<long>(i) * (NT / 8) * 2048);
  bf16x8 naf[8], nbf[8];
#pragma unroll
  for (int a = 0; a < 8; ++a) naf[a] = frag16(smem, wm + a * 16, 0, lane);
#pragma unroll
  for (int b = 0; b < 8; ++b) nbf[b] = frag16(smem + BM * BK, wn + b * 16, 0, lane);
  for (int ks = 0; ks < ksteps; ++ks) {
    const uint16_t* As = smem + (ks & 1) * STAGE;
    const uint16_t* Bs = As + BM * BK;
    uint16_t* Nx = smem + ((ks + 1) & 1) * STAGE;
    const uint16_t* gk = gp + ((ks + 2) % kRing) * 64;
    // the B half of a step: rows 256..511 of the stage = chunks i >= 8; 32 rows x 8 chunks per i
    const uint16_t* gb = cold + (static_cast<long>(blockIdx.x) * kStreamSteps + ((ks + 2) % kStreamSteps)) * kStreamStep +
                         row * 64 + chunk * 8;
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
      bf16x8 af[8], bf[8];
#pragma unroll
      for (int a = 0; a < 8; ++a) af[a] = naf[a];
#pragma unroll
      for (int b = 0; b < 8; ++b) bf[b] = nbf[b];
      if (kk == 0) {
#pragma unroll
        for (int a = 0; a < 8; ++a) naf[a] = frag16(As, wm + a * 16, 1, lane);
#pragma unroll
        for (int b = 0; b < 8; ++b) nbf[b] = frag16(Bs, wn + b * 16, 1, lane);
      }
#pragma unroll
      for (int i = kk * 8; i < kk * 8 + 8; ++i) {
        *reinterpret_cast<u32x4*>(Nx + lds0 + i * (NT / 8) * BK) = st[i];
        st[i] = (STREAM && i >= 8) ? *reinterpret_cast<const u32x4*>(gb + (i - 8) * 2048)
                                   : *reinterpret_cast<const u32x4*>(gk + static_cast<long>(i) * (NT / 8) * 2048);
      }
#pragma unroll
      for (int a = 0; a < 8; ++a)
#pragma unroll
        for (int b = 0; b < 8; ++b) acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[b], af[a], acc[a][b], 0, 0, 0);
    }
    __syncthreads();
#pragma unroll
    for (int a = 0; a < 8; ++a) naf[a] = frag16(Nx, wm + a * 16, 0, lane);
#pragma unroll
    for (int b = 0; b < 8; ++b) nbf[b] = frag16(Nx + BM * BK, wn + b * 16, 0, lane);
  }
  float s = 0.f;
  for (int a = 0; a < 8; ++a) for (int b = 0; b < 8; ++b) for (int i = 0; i < 4; ++i) s += acc[a][b][i];
  if (s == 12345.f) out[0] = s;
}

template <typename K>
bool allow_lds(K kernel) {
  return hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                             2 * STAGE * 2) == hipSuccess;
}

}  // namespace

// Elements (bf16) the two operand buffers must hold for `blocks` workgroups.
extern "C" long mi355_probe_kloop_hot_elems(int blocks) { return static_cast<long>(blocks) * (BM + BN) * 2048 / 16 + (BM + BN) * 2048l + 2 * STAGE; }
extern "C" long mi355_probe_kloop_cold_elems(int blocks) { return static_cast<long>(blocks) * kStreamSteps * kStreamStep; }

// One launch of `blocks` workgroups running `ksteps` K steps of variant 0..6 (see the head of this
// file).  placement 0: every workgroup re-reads its own 2 MiB window of `hot`, the windows 128 KiB
// apart (34 MB for 256 workgroups: more than the L2 of an XCD, within the memory-side cache);
// 1: the same, but the B half of every step streams from `cold` (variants 0..3 only); 2: all
// workgroups re-read one 2 MiB window (resident in every L2).  flops = blocks * ksteps * 2 * 256 *
// 256 * 64.  Returns 0, or a negative value for a bad argument / failed launch.
extern "C" int mi355_probe_kloop(int variant, int placement, const void* hot, const void* cold, float* sink,
                                 int blocks, int ksteps, void* stream) {
  if (!hot || !sink || blocks < 1 || ksteps < 1 || variant < 0 || variant > 6 || placement < 0 || placement > 2) return -1;
  const int stream_hbm = placement == 1;
  if (stream_hbm && (!cold || variant > 3)) return -1;
  const uint16_t* h = static_cast<const uint16_t*>(hot);
  const uint16_t* c = static_cast<const uint16_t*>(cold);
  const long stride = placement == 2 ? 0 : (BM + BN) * 2048l / 16;
  const size_t lds = 2 * STAGE * 2;
  hipStream_t s = static_cast<hipStream_t>(stream);
#define MI355_KLOOP(kernel, threads, ...)                                                  \
  do {                                                                                     \
    if (!allow_lds(kernel)) return -2;                                                     \
    hipLaunchKernelGGL(kernel, dim3(blocks), dim3(threads), lds, s, h, c, sink, ksteps, stride, ##__VA_ARGS__); \
  } while (0)
  if (variant == 0) { if (stream_hbm) MI355_KLOOP((kloop_product<1, 1>), 512, 4); else MI355_KLOOP((kloop_product<1, 0>), 512, 4); }
  if (variant == 1) { if (stream_hbm) MI355_KLOOP((kloop_product<0, 1>), 512, 4); else MI355_KLOOP((kloop_product<0, 0>), 512, 4); }
  if (variant == 2) { if (stream_hbm) MI355_KLOOP(kloop_direct<1>, 512); else MI355_KLOOP(kloop_direct<0>, 512); }
  if (variant == 3) { if (stream_hbm) MI355_KLOOP(kloop_four_waves<1>, 256); else MI355_KLOOP(kloop_four_waves<0>, 256); }
  if (variant == 4) MI355_KLOOP((kloop_product<0, 0, 0, 1>), 512, 4);
  if (variant == 5) MI355_KLOOP((kloop_product<0, 0, 1, 0>), 512, 4);
  if (variant == 6) MI355_KLOOP((kloop_product<0, 0, 0, 0>), 512, 4);
#undef MI355_KLOOP
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
