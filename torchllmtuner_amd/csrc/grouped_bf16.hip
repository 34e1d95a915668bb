// Grouped SwiGLU expert GEMMs in bf16 on the gfx950 matrix cores.
//
// Products (no transpose is ever materialised):
//   gate/up  rows . w1^T, rows . w3^T   A KC, B KC   fused SiLU*up epilogue
//   down     h . w2^T                   A KC, B KC
//   dh       dy . w2                    A KC, B KS   fused SwiGLU backward epilogue
//   drows    dgate . w1 + dup . w3      A KC, B KS   (one accumulator, K = 2F)
//   dw*      a_e^T . b_e                A KS, B KS   K = the expert's rows
//
// Shape of the kernels.  256x256 output tiles for the row-tiled products and the weight
// gradients alike, eight waves per workgroup as 4 (rows) x 2 (columns), two per SIMD, each
// wave a 64x128 accumulator tile; one workgroup per CU, two 64 KiB LDS stages of operand
// tiles (overlaid by the eight 17 KiB epilogue regions).  Row tiles come from the
// permutation plan's tile list (up to 256 rows of one expert each).
//
// What bounds them, measured on MI355X.  With operands of random bits the card's power
// management holds the core clock near 1.5-1.9 GHz (2.4 GHz with constant operands): a
// register-resident MFMA loop sustains 1.45-1.95 PFLOP/s instead of the 2.5 PFLOP/s of the
// data sheet, the same loop fed from LDS and staging its operands from L2 about 1.0-1.1.
// The K loops here run at that rate; operand traffic is not the limit (L2 delivers
// 50 B/clk/CU to a tile-shaped read pattern, HBM 10 B/clk/CU, and making every operand
// cache-resident changes nothing).  What is left is everything around the K loop, hence:
//   * persistent workgroups: block b serves XCD b % 8 and walks that XCD's contiguous
//     run of tiles with stride gridDim/8, so the tiles in flight on an XCD are
//     neighbours that share an expert's weights in its L2, and no workgroup launch sits
//     between two tiles;
//   * tile metadata looked up two tiles ahead, the first K step of the next tile
//     requested before the epilogue of the current one; the barrier between tiles waits
//     for LDS traffic only, so a tile's stores drain under the next tile's work;
//   * hardware bf16 conversion and transcendental-unit sigmoid in the epilogues (they
//     were VALU bound);
//   * a wave skips the MFMAs of 16-row blocks that hold no real rows (last tile of an
//     expert).
//
// K loop: one barrier per K step of 64.  Per quarter step a wave reads its fragments,
// parks a quarter of the next step's operands (held in registers) in the other LDS
// stage, refills those registers with the step after, and issues its MFMAs.  The
// pipeline tail is peeled at compile time: every load of the steady state is
// unconditional, so the compiler counts outstanding loads exactly instead of draining
// the queue once per K step.  Operands are fetched with buffer loads: a wave-uniform
// resource (the tile's origin), a fixed 32-bit per-thread offset and a scalar K offset,
// so no per-thread 64-bit address arithmetic or address registers sit in the loop.
//
// MFMA of the row-tiled kernels: v_mfma_f32_16x16x32_bf16.  Per lane 8 bf16 of each operand (row lane%16,
// k = 8*(lane/16)..+7), 4 fp32 of the result (column lane%16, rows 4*(lane/16) + i).
// With random operand bits this shape sustains about 14 % more than 32x32x16 on this
// card (2.17 against 1.90 PFLOP/s register-resident, +7 % in a whole K loop).  The weight tile is passed as the FIRST operand
// and the activation tile as the second, so a lane ends up with four CONSECUTIVE
// output columns of one output row: epilogues pack them and go through LDS to
// write 16-byte, fully coalesced rows.
//
// The LDS layouts (KC / KS) and fragment reads are in bf16_tiles.h.
#include <algorithm>
#include <cstdlib>
#include <type_traits>

#include "bf16_tiles.h"
#include "common.h"

namespace mi355 {
namespace {

constexpr int NT = 512;  // threads per workgroup

// 1 / (1 + e^-x) on the transcendental unit (v_exp_f32, v_rcp_f32: about 1 ulp each; every
// use is rounded to bf16 right after)
__device__ __forceinline__ float fast_sigmoid(float x) {
  return __builtin_amdgcn_rcpf(1.0f + __expf(-x));
}

// Raw buffer resource over `base` (wave-uniform): byte offsets up to 4 GiB, no stride, no
// swizzle; loads through it take a 32-bit per-thread offset and a scalar offset.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, -1, 0x00020000);
}

// int32 data that no kernel of this file writes (the plan's arrays), for uniform lookups
typedef const int32_t __attribute__((address_space(4))) * const_i32;

// RM_DLIN: the product of RM_DH (rows . w[e], the weight's contraction axis strided) with a plain epilogue:
// the input gradient of one grouped linear map
enum RowMode { RM_GATEUP = 0, RM_DOWN = 1, RM_DH = 2, RM_DX = 3, RM_DLIN = 4 };

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
  const int32_t* a_src;  // GATEUP, DH: row -> row of a0 to read (token gather), or null
  int a_rows;            // rows of a0 when a_src is given: gathered indices are clamped to [0, a_rows)
  // DH with a_src (the combine's backward folded in): a0 is the layer's output gradient (T, D),
  // row r stands for row_scale[r] * a0[a_src[r]]; o2 receives row_scale * h and dot_partial
  // [row][dot_slots] the pieces of <unscaled dh row, h row>, one per 128 output columns
  const float* row_scale;
  float* dot_partial;
  int dot_slots;
  const int32_t* seg_offsets;
  const int32_t* seg_counts;
  const int32_t* tile_expert;
  const int32_t* tile_row0;
  const int32_t* num_tiles;
  int D, F;
  int n_tiles;
};

// Row-tiled kernel: 64 WM rows of one expert x 32 NJ (8 / WM) output columns, 8 waves as WM
// (rows) x 8 / WM (columns), each wave 64 x 32 NJ.  GATEUP's columns are half gate and half
// up columns of the same f range, so a wave holds gate and up of the same 16 NJ f.

struct TileMeta {
  int e, row0, valid, n0, nt;
};

// sum over each group of 16 consecutive lanes, left in all 16 (DPP row operations)
__device__ __forceinline__ float row16_sum(float v) {
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0xB1, 0xf, 0xf, false));   // quad_perm [1,0,3,2]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x4E, 0xf, 0xf, false));   // quad_perm [2,3,0,1]
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x141, 0xf, 0xf, false));  // row_half_mirror
  v += __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), 0x140, 0xf, 0xf, false));  // row_mirror
  return v;
}

// SAVE_GU (GATEUP only): also write gate and up, which the backward reads; a forward-only caller
// leaves them out -- a third of the kernel's output bytes and of its epilogue's LDS traffic.
template <int MODE, int NJ, bool GATHER, int WM, bool SAVE_GU = true>
__global__ __launch_bounds__(NT, 2) void row_tiled_kernel(RowArgs p) {
  constexpr int WN = 8 / WM;               // waves along the columns (WM along the rows)
  constexpr int TBM = 64 * WM;             // rows of the tile
  constexpr int BNT = 32 * NJ * WN;        // output columns of the tile (WN waves x NJ x 32)
  constexpr int NA = TBM / 64;             // 16-byte A chunks staged per thread and K step
  constexpr int NB = BNT / 64;             // the same for B
  constexpr int STAGE = (TBM + BNT) * BK;  // elements per LDS stage
  constexpr bool DH_LIKE = (MODE == RM_DH || MODE == RM_DLIN);  // same operands, different epilogue
  constexpr bool B_KS = (DH_LIKE || MODE == RM_DX);
  static_assert(!GATHER || MODE == RM_GATEUP || MODE == RM_DH, "only gate/up and dH gather their rows");
  static_assert(!(GATHER && MODE == RM_DH) || NJ == 4, "the fused dH epilogue reduces over 16 lanes per row");
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave / WN) * 64, wn = wave % WN;
  const int wave_m = __builtin_amdgcn_readfirstlane(wm);  // the same value, known to be wave-uniform
  const int D = p.D, F = p.F;
  const int Kdim = (MODE == RM_GATEUP || DH_LIKE) ? D : (MODE == RM_DOWN ? F : 2 * F);
  const int lda = (MODE == RM_GATEUP || DH_LIKE) ? D : F;
  const int Ncols = (MODE == RM_GATEUP || DH_LIKE) ? F : D;  // output width
  const int64_t wsz = static_cast<int64_t>(D) * F;
  const int ksteps = Kdim / BK;

  // Persistent workgroups: block b serves XCD b % 8 and walks that XCD's contiguous run
  // of the tile list with stride gridDim/8, the order in which the hardware dispatcher
  // would have started one-tile blocks.  Tile metadata is looked up two tiles ahead and
  // the first operands of the next tile are requested before the epilogue of the current
  // one, so neither lookup nor first fetch sits between two K loops; a tile's stores
  // drain under the next tile's work.
  const int num_tiles = *p.num_tiles;
  const int total = num_tiles * p.n_tiles;
  const int chunk = (total + 7) >> 3;
  const int stride = gridDim.x >> 3;
  const int pid_base = (blockIdx.x & 7) * chunk;
  int within = blockIdx.x >> 3;
  if (within >= chunk || pid_base + within >= total) return;
  auto exists = [&](int w) { return w < chunk && pid_base + w < total; };
  auto load_meta = [&](int w) -> TileMeta {
    const int pid = pid_base + w;
    // scalar loads (constant address space): as vector loads these lookups would share the
    // counter of the operand stream and of the epilogue stores, and waiting for one of them
    // would wait for all of those
    const int t = pid / p.n_tiles;  // some tile of the expert this work item belongs to
    TileMeta m;
    m.e = ((const_i32)p.tile_expert)[t];
    const int cnt_e = ((const_i32)p.seg_counts)[m.e], off_e = ((const_i32)p.seg_offsets)[m.e];
    const int h = even_tile_rows(cnt_e, TBM);
    const int nrt = max((cnt_e + TBM - 1) / TBM, 1);  // row tiles of the expert
    // Within an expert the work items run column-tile-major over groups of three row tiles:
    // the row tiles of one column tile are neighbours, so the weight tile they share -- the
    // larger operand: an expert's weights are several times its rows -- is in L2 when the next
    // one asks for it, and a row tile's column tiles are still at most 3 x n_tiles work items
    // apart, inside what an XCD has in flight.  Row-tile-major throughout (neighbours share
    // the row tile only) left a quarter of the weight tiles to be fetched twice;
    // column-tile-major throughout fetches the rows of an expert with many row tiles once per
    // column tile.
    constexpr int G = 3;
    const int t0 = t - (((const_i32)p.tile_row0)[t] - off_e) / h;  // the expert's first tile
    const int q = pid - t0 * p.n_tiles;
    const int blk = q / (G * p.n_tiles);
    const int qb = q - blk * (G * p.n_tiles);
    const int g = min(G, nrt - blk * G);  // row tiles of this group (>= 1)
    const int nt = qb / g, rt = blk * G + (qb - nt * g);
    m.row0 = off_e + rt * h;
    m.valid = min(h, cnt_e - rt * h);
    // a last tile that would overhang starts early instead and recomputes a few columns
    // of its neighbour (same values), so no column is ever clamped
    constexpr int W = (MODE == RM_GATEUP ? BNT / 2 : BNT);
    m.n0 = min(nt * W, Ncols - W);
    m.nt = nt;
    return m;
  };

  // ---- global -> register staging: 16-byte chunks q = tid + 512*i ---------------------
  // KC tiles (8 chunks per row): row (tid>>3) + 64*i, chunk tid&7.
  // KS tile (BNT/8 chunks per k row): chunk q -> k = q / (BNT/8), chunk q % (BNT/8).
  u32x4 ra[NA], rb[NB];
  const int kc_row = tid >> 3, kc_chunk = tid & 7;
  const int kc_lds = kc_row * BK + ((kc_chunk ^ ((kc_row >> 1) & 7)) << 3);  // + i*64*BK (64 % 16 == 0)
  int b_lds[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    if constexpr (!B_KS) {
      b_lds[i] = kc_lds + i * 64 * BK;
    } else {
      constexpr int CPR = BNT / 8;  // chunks per k row
      const int q = tid + NT * i;
      const int k = q / CPR, cc = q % CPR;
      b_lds[i] = k * BNT + ((cc ^ ks_key16(k)) << 3);
    }
  }
  // a wave's 64 x (32 NJ) accumulator tile is 4 x NJ2 MFMA tiles of 16 x 16; with
  // gate/up the first NJ column tiles are gate columns, the last NJ the same f of up
  constexpr int NJ2 = 2 * NJ;
  int bcol[NJ2];
#pragma unroll
  for (int nj = 0; nj < NJ2; ++nj) {
    if constexpr (MODE == RM_GATEUP)
      bcol[nj] = (nj < NJ ? 0 : BNT / 2) + wn * (16 * NJ) + (nj % NJ) * 16;
    else
      bcol[nj] = wn * (32 * NJ) + nj * 16;
  }

  // Operand addresses are a wave-uniform buffer resource (the tile's origin) plus a fixed 32-bit
  // per-thread byte offset plus a scalar offset (K step, chunk round): the form buffer loads take
  // without any per-thread 64-bit arithmetic or address registers.  The B offsets never change;
  // the A offsets follow the tile's rows.
  constexpr bool B_REGULAR = !B_KS || (NT % (BNT / 8) == 0);  // chunk index -> fixed row stride
  constexpr int NBV = B_REGULAR ? 1 : NB;
  const int ldb = B_KS ? Ncols : (MODE == RM_GATEUP ? D : F);
  uint32_t voffB[NBV];
  if constexpr (!B_KS) {
    voffB[0] = static_cast<uint32_t>(kc_row * ldb + kc_chunk * 8) * 2u;
  } else {
    constexpr int CPR = BNT / 8;
#pragma unroll
    for (int i = 0; i < NBV; ++i) {
      const int q = tid + NT * i;
      voffB[i] = static_cast<uint32_t>((q / CPR) * ldb + (q % CPR) * 8) * 2u;
    }
  }
  // state of the tile whose operands are being fetched
  __amdgpu_buffer_rsrc_t rsA0, rsA1;  // A rows (k = 0); DX: second half of the contraction (dup)
  __amdgpu_buffer_rsrc_t rsB0, rsB1;  // B tile origin in the first / second weight stack
  uint32_t voffA[NA];
  // source rows of the A tile: the tile's own rows, or token rows through the gather index
  auto load_asrc = [&](const TileMeta& m, int (&asrc)[NA]) {
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int r = max(min(kc_row + 64 * i, m.valid - 1), 0);
      // (the index as loaded: it is clamped to [0, a_rows) where it is used, in setup(), a whole K
      // loop later, so that nothing waits for this load here)
      asrc[i] = GATHER ? p.a_src[m.row0 + r] : r;
    }
  };
  auto setup = [&](const TileMeta& m, const int (&asrc)[NA]) {
    const int64_t arow = GATHER ? 0 : static_cast<int64_t>(m.row0) * lda;
    rsA0 = make_rsrc(p.a0 + arow);
    rsA1 = (MODE == RM_DX) ? make_rsrc(p.a1 + arow) : rsA0;
#pragma unroll
    for (int i = 0; i < NA; ++i) {
      const int src = GATHER ? min(max(asrc[i], 0), p.a_rows - 1) : asrc[i];
      voffA[i] = (static_cast<uint32_t>(src) * static_cast<uint32_t>(lda) + static_cast<uint32_t>(kc_chunk * 8)) * 2u;
    }
    const uint16_t* B0 = p.b0 + m.e * wsz;
    const uint16_t* B1 = (MODE == RM_GATEUP || MODE == RM_DX) ? p.b1 + m.e * wsz : B0;
    // KC: the tile's first weight row is n0; KS: its first column is n0
    const int64_t borg = B_KS ? static_cast<int64_t>(m.n0) : static_cast<int64_t>(m.n0) * ldb;
    rsB0 = make_rsrc(B0 + borg);
    rsB1 = make_rsrc(B1 + borg);
  };
  // chunk i of the A / B tile of the K step that starts at k0
  auto load_a = [&](int k0, int i) -> u32x4 {
    if constexpr (MODE == RM_DX) {
      if (k0 >= F) return __builtin_amdgcn_raw_buffer_load_b128(rsA1, voffA[i], (k0 - F) * 2, 0);
    }
    return __builtin_amdgcn_raw_buffer_load_b128(rsA0, voffA[i], k0 * 2, 0);
  };
  auto load_b = [&](int k0, int i) -> u32x4 {
    if constexpr (MODE == RM_GATEUP) {
      // rows 0..BNT/2 of the tile come from w1, the rest from w3, same f range
      const int so = (64 * (i % (NB / 2)) * ldb + k0) * 2;
      return __builtin_amdgcn_raw_buffer_load_b128(i >= NB / 2 ? rsB1 : rsB0, voffB[0], so, 0);
    } else if constexpr (MODE == RM_DOWN) {
      return __builtin_amdgcn_raw_buffer_load_b128(rsB0, voffB[0], (64 * i * ldb + k0) * 2, 0);
    } else {
      int kk0 = k0;
      bool second = false;
      if constexpr (MODE == RM_DX) {
        if (k0 >= F) { kk0 = k0 - F; second = true; }
      }
      const int so = (kk0 + (B_REGULAR ? i * (NT / (BNT / 8)) : 0)) * ldb * 2;
      return __builtin_amdgcn_raw_buffer_load_b128(second ? rsB1 : rsB0, voffB[B_REGULAR ? 0 : i], so, 0);
    }
  };
  auto kofs = [&](int ks) { return ks * BK; };
  // request every chunk of K step `step` of the fetch tile
  // (chunk after chunk in the order of a K step of the loop below, and kept in that order: the
  // loop's waits count the requests that follow the one they need along every way into the loop,
  // so every way must issue them alike -- with all A chunks first the park of the first B chunk
  // waited for five requests more than it needed)
  auto issue = [&](int step) {
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      __builtin_amdgcn_sched_barrier(0);
      if (q < NA) ra[q] = load_a(kofs(step), q);
#pragma unroll
      for (int i = (q * NB) / 4; i < ((q + 1) * NB) / 4; ++i) rb[i] = load_b(kofs(step), i);
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  TileMeta cur = load_meta(within);
  TileMeta nxt = load_meta(exists(within + stride) ? within + stride : within);
  {
    int asrc[NA];
    load_asrc(cur, asrc);
    setup(cur, asrc);
    issue(0);
  }

  for (;;) {
  const bool more = exists(within + stride);
  // the tile after the next: looked up now, used one tile later
  const TileMeta nxt2 = load_meta(exists(within + 2 * stride) ? within + 2 * stride : within);
  int nsrc[NA];
  load_asrc(nxt, nsrc);
  const int row0 = cur.row0, valid = cur.valid, n0 = cur.n0, ntile = cur.nt;

  f32x4 acc[4][NJ2];
#pragma unroll
  for (int mi = 0; mi < 4; ++mi)
#pragma unroll
    for (int nj = 0; nj < NJ2; ++nj)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[mi][nj][i] = 0.0f;

  // K step 0 (requested before the previous epilogue) -> LDS stage 0, K step 1 -> registers
#pragma unroll
  for (int i = 0; i < NA; ++i) *reinterpret_cast<u32x4*>(smem + kc_lds + i * 64 * BK) = ra[i];
#pragma unroll
  for (int i = 0; i < NB; ++i) *reinterpret_cast<u32x4*>(smem + TBM * BK + b_lds[i]) = rb[i];
  if (ksteps > 1) issue(1);
  __syncthreads();

  // One K step.  HAS_NEXT: the registers hold tile ks+1 and are parked in the other LDS
  // stage.  HAS_NEXT2: tile ks+2 is fetched into the registers.  Both are compile-time
  // so that every load of the steady-state loop is unconditional: the compiler can then
  // count outstanding loads exactly and wait only for the three oldest before each park,
  // instead of draining the queue (vmcnt(0)) once per K step.
  // The last tile of an expert is partly empty: a wave skips the MFMAs of its 16-row
  // blocks that hold no real rows (a wave-uniform branch; operands are still staged and
  // every barrier met).
  const int act = min(max((valid - wave_m + 15) >> 4, 0), 4);
  auto kstep = [&](int ks, auto has_next_t, auto has_next2_t) {
    constexpr bool has_next = decltype(has_next_t)::value;
    constexpr bool has_next2 = decltype(has_next2_t)::value;
    const uint16_t* As = smem + (ks & 1) * STAGE;
    const uint16_t* Bs = As + TBM * BK;
    uint16_t* An = smem + ((ks + 1) & 1) * STAGE;
    uint16_t* Bn = An + TBM * BK;
#pragma unroll
    for (int kk = 0; kk < BK / 32; ++kk) {
      bf16x8 af[4];
#pragma unroll
      for (int mi = 0; mi < 4; ++mi) af[mi] = frag16_kc(As, wm + mi * 16, kk, lane);
#pragma unroll
      for (int hb = 0; hb < 2; ++hb) {
        bf16x8 bf[NJ];
#pragma unroll
        for (int b = 0; b < NJ; ++b) {
          if constexpr (B_KS)
            bf[b] = frag16_ks<BNT>(Bs, bcol[hb * NJ + b], kk, lane);
          else
            bf[b] = frag16_kc(Bs, bcol[hb * NJ + b], kk, lane);
        }
        // a quarter of the staging traffic rides along with each quarter of the MFMAs:
        // park the held chunks of tile ks+1 in the other LDS stage, then refill the
        // same registers with the same chunks of tile ks+2.
        const int q = kk * 2 + hb;
        if constexpr (has_next) {
          // A: two chunks ride with the first two quarters, or one with each of the four
          if (q < NA) *reinterpret_cast<u32x4*>(An + kc_lds + q * 64 * BK) = ra[q];
#pragma unroll
          for (int i = (q * NB) / 4; i < ((q + 1) * NB) / 4; ++i)
            *reinterpret_cast<u32x4*>(Bn + b_lds[i]) = rb[i];
        }
        if constexpr (has_next2) {
          if (q < NA) ra[q] = load_a(kofs(ks + 2), q);
#pragma unroll
          for (int i = (q * NB) / 4; i < ((q + 1) * NB) / 4; ++i) rb[i] = load_b(kofs(ks + 2), i);
        }
#pragma unroll
        for (int mi = 0; mi < 4; ++mi) {
          if (mi < act) {
#pragma unroll
            for (int b = 0; b < NJ; ++b)
              acc[mi][hb * NJ + b] =
                  __builtin_amdgcn_mfma_f32_16x16x32_bf16(bf[b], af[mi], acc[mi][hb * NJ + b], 0, 0, 0);
          }
        }
      }
    }
    __syncthreads();
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  int ks = 0;
  for (; ks + 2 < ksteps; ++ks) kstep(ks, T_{}, T_{});
  if (ks + 1 < ksteps) { kstep(ks, T_{}, F_{}); ++ks; }
  if (ks < ksteps) kstep(ks, F_{}, F_{});

  // switch the fetch state to the next tile and request its first K step: the loads
  // are in flight while the epilogue below runs
  if (more) {
    setup(nxt, nsrc);
    issue(0);
  }

  // ---- epilogue: through the wave's private LDS region, 16-byte coalesced rows ---------
  // acc[mi][nj][i]: output row = wm + mi*16 + (lane&15); output column within the nj-th
  // 16-column tile = 4*(lane>>4) + i.
  uint16_t* st = smem + wave * (64 * 136);  // 8 waves x 17 KiB < 160 KiB; the barrier ending the K loop freed the tiles
  if constexpr (MODE == RM_GATEUP) {
    // per 32-row half: three 32 x 64 tiles gate | up | h at columns 0, 64, 128 of a
    // [32][192+8] region (12.5 KiB per wave); without gate and up, h alone in a [32][64+8] region
    constexpr int NT3 = SAVE_GU ? 3 : 1;       // output tiles per row
    using S = WaveStage<64 * NT3>;
    uint16_t* sg = smem + wave * (32 * S::PITCH);
    const int f0 = n0 + wn * 64;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      if (wave_m + half * 32 >= valid) continue;  // no real rows in this half (uniform per wave)
#pragma unroll
      for (int ml = 0; ml < 2; ++ml)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const int mi = half * 2 + ml;
          float g[4], u[4], h[4];
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            g[r] = round_bf16(acc[mi][j][r]);
            u[r] = round_bf16(acc[mi][j + NJ][r]);
            const float s = round_bf16(g[r] * fast_sigmoid(g[r]));
            h[r] = s * u[r];
          }
          if constexpr (SAVE_GU) {
            S::put16(sg, ml, j * 16, lane, g[0], g[1], g[2], g[3]);
            S::put16(sg, ml, 64 + j * 16, lane, u[0], u[1], u[2], u[3]);
          }
          S::put16(sg, ml, (SAVE_GU ? 128 : 0) + j * 16, lane, h[0], h[1], h[2], h[3]);
        }
      __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): the wave's own LDS writes have landed
      __builtin_amdgcn_wave_barrier();
      // 32 rows x NT3 tiles x 8 chunks, 4 NT3 per lane
#pragma unroll 4
      for (int it = 0; it < 4 * NT3; ++it) {
        const int idx = it * 64 + lane;
        const int m = idx / (8 * NT3), rem = idx % (8 * NT3), t = rem >> 3, c = rem & 7;
        const int f = f0 + c * 8;  // < F: tiles never overhang in the columns
        const int mr = wm + half * 32 + m;
        if (mr < valid) {
          const u32x4 v = *reinterpret_cast<const u32x4*>(sg + m * S::PITCH + t * 64 + c * 8);
          uint16_t* dst = (!SAVE_GU ? p.o2 : (t == 0 ? p.o0 : (t == 1 ? p.o1 : p.o2))) + static_cast<int64_t>(row0 + mr) * F + f;
          *reinterpret_cast<u32x4*>(dst) = v;
        }
      }
      __builtin_amdgcn_s_waitcnt(0xc07f);
      __builtin_amdgcn_wave_barrier();
    }
  } else if (wave_m < valid) {
    using S = WaveStage<32 * NJ>;
    constexpr int CH = 4 * NJ;  // 16-byte chunks per row of the wave's sub-tile
#pragma unroll
    for (int mi = 0; mi < 4; ++mi)
#pragma unroll
      for (int nj = 0; nj < NJ2; ++nj)
        S::put16(st, mi, nj * 16, lane, acc[mi][nj][0], acc[mi][nj][1], acc[mi][nj][2], acc[mi][nj][3]);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    const int c0 = n0 + wn * (32 * NJ);
    // 64 rows x CH chunks, CH per lane; a row's bytes go out contiguously; tiles never
    // overhang in the columns.  Where the epilogue also LOADS (dH), lanes whose row lies past
    // the tile's real rows redo the last real row instead (the same bytes to the same
    // address), so that every load and store is unconditional: the compiler then knows how
    // many are in flight and waits for exactly the ones it needs -- with predicated accesses
    // every wait drains the whole queue, stores included (one counter serves both here).
    const int last = valid - 1 - wm;  // >= 0 in this branch
    auto chunk_at = [&](int it, int& m, int& c) {
      const int idx = it * 64 + lane;
      m = min(idx / CH, last);
      c = idx % CH;
    };
    auto offset_at = [&](int it) -> int64_t {
      int m, c;
      chunk_at(it, m, c);
      return static_cast<int64_t>(row0 + wm + m) * Ncols + c0 + c * 8;
    };
    if constexpr (MODE == RM_DH) {
      // SwiGLU backward on 8 consecutive f: dgate = dh*up*silu'(gate), dup = dh*silu(gate).
      // gate and up of the next four chunks are requested before the current four are stored:
      // a load issued behind a store cannot complete before it.
      // With the combine's backward folded in (FUSE), the staged value is the unscaled dh row:
      // its product with the row's h (recomputed from gate and up) summed over f is the
      // gradient of the row's routing score, reduced here over the 16 lanes that share a row
      // and written once per row and 128-column slot; dh itself is then scaled by the score,
      // and score * h goes out as the operand of the dW2 product.
      constexpr bool FUSE = GATHER;
      constexpr int G = 4;
      static_assert(CH % G == 0, "chunks per row come in groups of four");
      auto row_at = [&](int it) -> int {
        int m, c;
        chunk_at(it, m, c);
        return row0 + wm + m;
      };
      u32x4 gq[G], uq[G];
      float sq[G];
#pragma unroll
      for (int u = 0; u < G; ++u) {
        const int64_t o = offset_at(u);
        gq[u] = *reinterpret_cast<const u32x4*>(p.gate + o);
        uq[u] = *reinterpret_cast<const u32x4*>(p.up + o);
        if constexpr (FUSE) sq[u] = p.row_scale[row_at(u)];
      }
#pragma unroll
      for (int g0 = 0; g0 < CH; g0 += G) {
        u32x4 gn[G], un[G];
        float sn[G];
        if (g0 + G < CH) {
#pragma unroll
          for (int u = 0; u < G; ++u) {
            const int64_t o = offset_at(g0 + G + u);
            gn[u] = *reinterpret_cast<const u32x4*>(p.gate + o);
            un[u] = *reinterpret_cast<const u32x4*>(p.up + o);
            if constexpr (FUSE) sn[u] = p.row_scale[row_at(g0 + G + u)];
          }
        }
#pragma unroll
        for (int u = 0; u < G; ++u) {
          int m, c;
          chunk_at(g0 + u, m, c);
          const u32x4 v = *reinterpret_cast<const u32x4*>(st + m * S::PITCH + c * 8);
          const u32x4 gv = gq[u], uv = uq[u];
          const float sc = FUSE ? sq[u] : 1.0f;
          float dot = 0.0f;
          u32x4 dg, du, hs;
#pragma unroll
          for (int w = 0; w < 4; ++w) {
            float r_dg[2], r_du[2], r_hs[2];
#pragma unroll
            for (int hlf = 0; hlf < 2; ++hlf) {
              float dh = __uint_as_float(hlf ? (v[w] & 0xffff0000u) : (v[w] << 16));
              const float g = __uint_as_float(hlf ? (gv[w] & 0xffff0000u) : (gv[w] << 16));
              const float uu = __uint_as_float(hlf ? (uv[w] & 0xffff0000u) : (uv[w] << 16));
              const float sig = fast_sigmoid(g);
              const float sl = round_bf16(g * sig);
              if constexpr (FUSE) {
                const float hv = round_bf16(sl * uu);  // h as the forward stored it
                dot += dh * hv;
                r_hs[hlf] = sc * hv;
                dh *= sc;
              }
              const float ds = round_bf16(dh * uu);
              r_du[hlf] = dh * sl;
              r_dg[hlf] = ds * (sig * (1.0f + g * (1.0f - sig)));
            }
            dg[w] = pack2(r_dg[0], r_dg[1]);
            du[w] = pack2(r_du[0], r_du[1]);
            if constexpr (FUSE) hs[w] = pack2(r_hs[0], r_hs[1]);
          }
          const int64_t o = offset_at(g0 + u);
          *reinterpret_cast<u32x4*>(p.o0 + o) = dg;
          *reinterpret_cast<u32x4*>(p.o1 + o) = du;
          if constexpr (FUSE) {
            *reinterpret_cast<u32x4*>(p.o2 + o) = hs;
            // columns below the tile's nominal start belong to its neighbour (a last tile
            // that would overhang starts early): they must not be counted twice
            if (c0 + c * 8 < ntile * BNT) dot = 0.0f;
            const float total = row16_sum(dot);
            // all 16 lanes of the row store the same value to the same address (unconditional,
            // like every other access of this epilogue)
            p.dot_partial[static_cast<int64_t>(row0 + wm + m) * p.dot_slots + ntile * WN + wn] = total;
          }
        }
        if (g0 + G < CH) {
#pragma unroll
          for (int u = 0; u < G; ++u) {
            gq[u] = gn[u];
            uq[u] = un[u];
            if constexpr (FUSE) sq[u] = sn[u];
          }
        }
      }
    } else {
      // plain copies, unconditional as well: lanes past the last real row store that row again
      // (same bytes, same address; the line is still in L2), so the stores are countable and
      // the next tile's first operands are not held up behind them (0.3 % per step; with an
      // expert's tiles equally tall a tile is rarely less than half full)
#pragma unroll 4
      for (int it = 0; it < CH; ++it) {
        const int idx = it * 64 + lane;
        const int m = min(idx / CH, last), c = idx % CH;
        *reinterpret_cast<u32x4*>(p.o0 + static_cast<int64_t>(row0 + wm + m) * Ncols + c0 + c * 8) =
            *reinterpret_cast<const u32x4*>(st + m * S::PITCH + c * 8);
      }
    }
  }
  // every wave is done with its staging region before the next tile's operands are parked;
  // only LDS traffic is waited for, the tile's stores keep draining
  phase_barrier();
  if (!more) break;
  within += stride;
  cur = nxt;
  nxt = nxt2;
  }
}

// ---- weight gradients: C[e](M,N) = sum_{r in segment e} A[r][m] * B[r][n] ----------
// 256 x 256 output tile, 8 waves as 4 (m) x 2 (n), each wave 64 x 128; both operands KS.
constexpr int WBM = 256, WBN = 256;
constexpr int W_STAGE = (WBM + WBN) * BK;  // 64 KiB

struct WgradArgs {
  const uint16_t* a;  // (rows, M) row-major
  const uint16_t* b;  // (rows, N) row-major
  uint16_t* c;        // (El, M, N)
  const int32_t* a_src;  // row -> row of a to read, or null (GATHER_A)
  const int32_t* b_src;  // row -> row of b to read (token gather), or null
  int src_rows;          // rows of the gathered operand: indices are clamped to [0, src_rows)
  const int32_t* seg_offsets;
  const int32_t* seg_counts;  // (2 El): row counts, then the local experts by descending count
  int El;
  int M, N;
  int m_tiles, n_tiles;
  int total;  // El * m_tiles * n_tiles
};

template <bool GATHER, bool GATHER_A = false>
__global__ __launch_bounds__(NT, 2) void wgrad_kernel(WgradArgs p) {
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 128;
  const int M = p.M, N = p.N;
  const int per_e = p.m_tiles * p.n_tiles;

  // KS tiles of 256 columns = 32 chunks per k row: k = (tid>>5) + 16*i, chunk tid&31
  u32x4 ra[4], rb[4];
  const int ks_k = tid >> 5, ks_chunk = tid & 31;
  int lds_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int k = ks_k + 16 * i;
    lds_off[i] = k * 256 + ((ks_chunk ^ ks_key(k)) << 3);
  }
  const u32x4 zero = {0, 0, 0, 0};

  // Persistent workgroups.  A tile's cost is its expert's row count (the contraction
  // length), which a skewed router spreads over two orders of magnitude, so tiles are not
  // walked in expert order: experts are taken by descending row count (the plan's order,
  // second half of seg_counts) and dealt to the eight XCDs a round at a time, and the CUs of an
  // XCD deal that XCD's tiles round-robin among themselves -- the longest contractions
  // start first and in parallel, and an expert's tiles still share one L2.  The K extent
  // is short for a balanced router (a handful of 64-row steps), so what surrounds the K
  // loop matters too: the first operands of the next tile are requested before the
  // epilogue of the current one and land while it runs, segment bounds are looked up
  // ahead, and with a gathered B operand the row indices of a K step are fetched one step
  // before its data.
  const int El = p.El;
  const int xcd = blockIdx.x & 7;
  // The plan arrays are read-only here and every lookup is workgroup-uniform: read through
  // the constant address space they are scalar loads.  As vector loads (what the compiler
  // makes of them inside this loop) each lookup would share the counter of the operand
  // stream and of the epilogue stores, and waiting for it would wait for all of those.
  const const_i32 order = (const_i32)(p.seg_counts + El);
  const const_i32 seg_offsets = (const_i32)p.seg_offsets;
  const const_i32 seg_counts = (const_i32)p.seg_counts;
  // Whole experts are dealt in rounds of eight, each round in the opposite direction of the
  // one before (so no XCD always gets the larger expert of its round); the El % 8 smallest
  // experts left over are cut into eight equal contiguous runs of tiles instead.
  const int n_full = (El >> 3) * per_e;
  const int pool = (El & 7) * per_e;
  const int p0 = static_cast<int>(static_cast<int64_t>(pool) * xcd >> 3);
  const int p1 = static_cast<int>(static_cast<int64_t>(pool) * (xcd + 1) >> 3);
  const int n_x = n_full + (p1 - p0);  // tiles of this XCD
  const int stride = gridDim.x >> 3;
  int within = blockIdx.x >> 3;
  if (within >= n_x) return;
  auto exists = [&](int w) { return w < n_x; };
  // this XCD's w-th tile (w clamped to an existing tile) as rank * per_e + tile in expert
  auto flat_of = [&](int w) -> int {
    w = exists(w) ? w : within;
    if (w >= n_full) return 8 * n_full + p0 + (w - n_full);
    const int round = w / per_e;
    return (round * 8 + ((round & 1) ? 7 - xcd : xcd)) * per_e + (w - round * per_e);
  };
  // (clamped: an order array the caller never filled must not turn into a wild address)
  auto expert_at = [&](int flat) -> int { return min(max(order[flat / per_e], 0), El - 1); };
  auto expert_of = [&](int w) -> int { return expert_at(flat_of(w)); };
  auto tile_in_expert = [&](int w) -> int { return flat_of(w) % per_e; };

  // state of the tile whose operands are being fetched
  int e = expert_of(within);
  // a last tile that would overhang starts early instead (M, N >= 256) and recomputes a few
  // rows or columns of its neighbour -- the same values -- so every tile is whole
  int m0 = min((tile_in_expert(within) / p.n_tiles) * WBM, M - WBM);
  int n0 = min((tile_in_expert(within) % p.n_tiles) * WBN, N - WBN);
  int seg0 = seg_offsets[e], cnt = seg_counts[e];
  const uint16_t* a_base;
  const uint16_t* b_base;
  auto set_bases = [&]() {
    a_base = p.a + (GATHER_A ? 0 : static_cast<int64_t>(seg0) * M) + min(m0 + ks_chunk * 8, M - 8);
    b_base = p.b + (GATHER ? 0 : static_cast<int64_t>(seg0) * N) + min(n0 + ks_chunk * 8, N - 8);
  };
  // B row of this thread's chunk i in K step `step` of segment (s0, c): its own row, or
  // (gather) the source row from the index array.  Needs c > 0.
  // (a gathered index is returned as loaded and clamped to [0, src_rows) only where it is used,
  // a K step later: clamping here would make the wave wait for the index right away, and with it
  // -- the load counter retires in order -- for every operand load requested before it)
  auto row_index = [&](int s0, int c, int step, int i) -> int {
    const int k = min(step * BK + ks_k + 16 * i, c - 1);
    return GATHER ? p.b_src[s0 + k] : k;
  };
  // the same for the A row (its own row unless A is gathered too)
  auto a_row_index = [&](int s0, int c, int step, int i) -> int {
    const int k = min(step * BK + ks_k + 16 * i, c - 1);
    return GATHER_A ? p.a_src[s0 + k] : k;
  };
  auto clamp_src = [&](int r) -> int { return min(max(r, 0), p.src_rows - 1); };
  // Loads of one K step, unconditional: rows past the segment re-read its last row and
  // the A side is zeroed when it is parked, so the products vanish.  Needs cnt > 0.
  auto load_ab = [&](int step, int i, int brow, int arow_g) {
    const int k = GATHER_A ? clamp_src(arow_g) : min(step * BK + ks_k + 16 * i, cnt - 1);
    const int kb = GATHER ? clamp_src(brow) : brow;
    ra[i] = *reinterpret_cast<const u32x4*>(a_base + static_cast<int64_t>(k) * M);
    rb[i] = *reinterpret_cast<const u32x4*>(b_base + static_cast<int64_t>(kb) * N);
  };
  auto park = [&](int step, int i, uint16_t* An, uint16_t* Bn, int count) {
    const bool live = step * BK + ks_k + 16 * i < count;
    *reinterpret_cast<u32x4*>(An + lds_off[i]) = live ? ra[i] : zero;
    *reinterpret_cast<u32x4*>(Bn + lds_off[i]) = rb[i];
  };
  int bidx[4];  // B rows of the K step that is requested next
  int aidx[4];  // A rows likewise (used when A is gathered)
  set_bases();
  if (cnt > 0) {
    // (requests always go out as operands, then the next index, chunk after chunk: the K loop's
    // waits count the requests that follow the one they need along every way into the loop)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      __builtin_amdgcn_sched_barrier(0);
      load_ab(0, i, row_index(seg0, cnt, 0, i), a_row_index(seg0, cnt, 0, i));
      bidx[i] = row_index(seg0, cnt, 1, i);
      aidx[i] = a_row_index(seg0, cnt, 1, i);
    }
    __builtin_amdgcn_sched_barrier(0);
  }
  // expert and segment of the next tile, expert of the one after it (its segment is
  // looked up inside the loop, the expert after that too)
  int ne = expert_of(within + stride);
  int nseg0 = seg_offsets[ne], ncnt = seg_counts[ne];
  int e2 = expert_of(within + 2 * stride);

  for (;;) {
    const bool more = exists(within + stride);
    const int nw = within + stride;
    // two tiles ahead: segment bounds, used one tile later; three ahead: the expert
    const int n2seg0 = seg_offsets[e2], n2cnt = seg_counts[e2];
    const int e3 = expert_of(within + 3 * stride);
    // next tile: B rows of its first K step (its bounds were looked up a tile ago)
    int nidx[4], nidx_a[4];
    if (ncnt > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        nidx[i] = row_index(nseg0, ncnt, 0, i);
        nidx_a[i] = a_row_index(nseg0, ncnt, 0, i);
      }
    }
    const int c_e = e, c_m0 = m0, c_n0 = n0, c_cnt = cnt, c_seg0 = seg0;
    const int ksteps = (cnt + BK - 1) / BK;

    // 64 x 128 per wave as 2 x 4 tiles of v_mfma_f32_32x32x16_bf16: with both operands read
    // through LDS transposes the 16x16x32 shape of the row-tiled kernels measured slower here
    f32x16 acc[2][4];
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int nj = 0; nj < 4; ++nj)
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[mi][nj][i] = 0.0f;

    if (ksteps > 0) {
#pragma unroll
      for (int i = 0; i < 4; ++i) park(0, i, smem, smem + WBM * BK, c_cnt);
      if (ksteps > 1) {
        // in the order of a K step of the loop below (operands, then the next index, chunk after
        // chunk, and kept in that order): the loop's waits count the requests that follow the one
        // they need, on both ways into the loop, so both ways must issue them alike
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          load_ab(1, i, bidx[i], aidx[i]);
          bidx[i] = row_index(c_seg0, c_cnt, 2, i);
          aidx[i] = a_row_index(c_seg0, c_cnt, 2, i);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();

    // One K step: a quarter of the staging rides along with each quarter of the MFMAs.
    // The flags are compile-time so that the loads of the steady state are unconditional
    // and the compiler counts outstanding loads exactly.
    auto kstep = [&](int ks, auto has_next_t, auto has_next2_t) {
      constexpr bool has_next = decltype(has_next_t)::value;
      constexpr bool has_next2 = decltype(has_next2_t)::value;
      const uint16_t* As = smem + (ks & 1) * W_STAGE;
      const uint16_t* Bs = As + WBM * BK;
      uint16_t* An = smem + ((ks + 1) & 1) * W_STAGE;
      uint16_t* Bn = An + WBM * BK;
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        // the last K step of a segment is usually ragged: its 16-row slices past the last real
        // row hold zeros and are skipped (workgroup-uniform; only this instantiation branches)
        if constexpr (!has_next) {
          if (ks * BK + kk * 16 >= c_cnt) continue;
        }
        bf16x8 af[2], bf[4];
#pragma unroll
        for (int mi = 0; mi < 2; ++mi) af[mi] = frag_ks<256>(As, wm + mi * 32, kk, lane);
#pragma unroll
        for (int nj = 0; nj < 4; ++nj) bf[nj] = frag_ks<256>(Bs, wn + nj * 32, kk, lane);
        if constexpr (has_next) park(ks + 1, kk, An, Bn, c_cnt);
        // Nothing is moved across this point: the requests below stay in their quarter of the K
        // step (left alone, the compiler gathers all of a step's global loads at its end, where
        // the data they fetch is parked a moment later instead of a whole step later, and the
        // wave waits out the memory latency once per K step), and an index is clamped a whole
        // step after it was requested.  What lies between two such points -- this quarter's
        // requests and MFMAs, the next quarter's fragment reads and its park -- is still
        // interleaved freely.
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (has_next2) {
          load_ab(ks + 2, kk, bidx[kk], aidx[kk]);
          bidx[kk] = row_index(c_seg0, c_cnt, ks + 3, kk);
          aidx[kk] = a_row_index(c_seg0, c_cnt, ks + 3, kk);
        }
#pragma unroll
        for (int mi = 0; mi < 2; ++mi)
#pragma unroll
          for (int nj = 0; nj < 4; ++nj)
            acc[mi][nj] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bf[nj], af[mi], acc[mi][nj], 0, 0, 0);
      }
      __syncthreads();
    };
    using T_ = std::true_type;
    using F_ = std::false_type;
    int ks = 0;
    for (; ks + 2 < ksteps; ++ks) kstep(ks, T_{}, T_{});
    if (ks + 1 < ksteps) { kstep(ks, T_{}, F_{}); ++ks; }
    if (ks < ksteps) kstep(ks, F_{}, F_{});

    // switch the fetch state to the next tile and request its first K step
    if (more) {
      e = ne;
      const int nt = tile_in_expert(nw);
      m0 = min((nt / p.n_tiles) * WBM, M - WBM);
      n0 = min((nt % p.n_tiles) * WBN, N - WBN);
      seg0 = nseg0;
      cnt = ncnt;
      set_bases();
      if (cnt > 0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          __builtin_amdgcn_sched_barrier(0);
          load_ab(0, i, nidx[i], nidx_a[i]);
          bidx[i] = row_index(seg0, cnt, 1, i);
          aidx[i] = a_row_index(seg0, cnt, 1, i);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }

    using S = WaveStage<128>;
    uint16_t* st = smem + wave * S::ELEMS;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi)
#pragma unroll
      for (int nj = 0; nj < 4; ++nj)
#pragma unroll
        for (int q = 0; q < 4; ++q)
          S::put4(st, mi, nj * 32, lane, q, acc[mi][nj][q * 4], acc[mi][nj][q * 4 + 1],
                  acc[mi][nj][q * 4 + 2], acc[mi][nj][q * 4 + 3]);
    __builtin_amdgcn_s_waitcnt(0xc07f);
    __builtin_amdgcn_wave_barrier();
    uint16_t* C = p.c + static_cast<int64_t>(c_e) * M * N;
#pragma unroll 4
    for (int it = 0; it < 16; ++it) {
      const int idx = it * 64 + lane;
      const int m = c_m0 + wm + (idx >> 4), n = c_n0 + wn + (idx & 15) * 8;
      // whole tiles only: the stores are unconditional, so the compiler knows how many follow
      // the operand loads requested above and the next tile's wait for those loads does not
      // also wait for these stores (one counter serves both)
      // (non-temporal: a weight gradient is several times the size of L2 and is read next by the
      // optimizer; written through the cache as ordinary stores, an expert's 30-60 MB of results push
      // its own operands out of L2 between two of its tiles -- with few rows per expert, where the
      // product is bound by these writes, the gathered rows were fetched from memory several times over)
      __builtin_nontemporal_store(*reinterpret_cast<const u32x4*>(st + (idx >> 4) * S::PITCH + (idx & 15) * 8),
                                  reinterpret_cast<u32x4*>(C + static_cast<int64_t>(m) * N + n));
    }
    // staging regions are free again before the next tile's operands are parked; only
    // the LDS traffic is waited for, the tile's stores keep draining
    phase_barrier();
    if (!more) break;
    within += stride;
    ne = e2;
    e2 = e3;
    nseg0 = n2seg0;
    ncnt = n2cnt;
  }
}

template <typename K>
int set_lds(K kernel, int bytes) {
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  return e == hipSuccess ? MI355_OK : fail(MI355_ELAUNCH, "hipFuncSetAttribute: %s", hipGetErrorString(e));
}

}  // namespace

// The MFMA path needs whole 64-wide K steps, 16-byte aligned rows, and outputs at least
// one tile wide (a last tile that would overhang is shifted back, never clamped).
int bf16_row_tile_m() { return 256; }

// ... and one expert's weight matrix below 2 GiB: operand loads address a tile with 32-bit byte offsets.
bool bf16_fast_path_ok(int64_t D, int64_t F) {
  return D % 64 == 0 && F % 64 == 0 && D >= 384 && F >= 384 && D * F < (1ll << 30);
}

enum { STAGE_GATEUP = 1, STAGE_DOWN = 2, STAGE_DH = 4, STAGE_DX = 8, STAGE_DW2 = 16, STAGE_DW1 = 32, STAGE_DW3 = 64 };

static unsigned round8(int64_t v) { return static_cast<unsigned>((v + 7) / 8 * 8); }

// One workgroup per CU (a workgroup takes the whole LDS), rounded to whole XCD rounds.
static unsigned resident_blocks() {
  static unsigned n = 0;
  if (n == 0) {
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus < 8)
      cus = 256;
    n = static_cast<unsigned>(cus / 8 * 8);
  }
  return n;
}

constexpr int W_LDS_BYTES = 8 * 64 * 136 * 2;  // 139264: the 8 epilogue regions (> 2 stages = 131072)

// width: output columns; gate/up tiles hold both halves of their column range.  Tiles are always
// 256 wide (a 192-wide KS tile would not hold the swizzle: 24 chunks per row are not a multiple
// of the 16 the key permutes); an overhanging last tile shifts back.
template <int MODE, bool GATHER = false, bool SAVE_GU = true>
static int launch_row(RowArgs& a, int64_t width, int64_t tile_capacity, hipStream_t s, const char* what) {
  constexpr int div = MODE == RM_GATEUP ? 2 : 1;
  a.n_tiles = (int)((width + 256 / div - 1) / (256 / div));
  // A product with so few row tiles that 256-column tiles would leave a quarter of the CUs or more without work
  // (the dH of one dense segment: 4096 rows x 2048 columns are 16 x 8 tiles) runs on 128-column
  // tiles instead: twice the work items, each with the whole contraction.  Only where the
  // epilogue does not depend on the tile width (the folded dH writes one partial per 128
  // columns of a 256-column tile).
  if constexpr ((MODE == RM_DH || MODE == RM_DLIN) && !GATHER) {
    if (tile_capacity * a.n_tiles * 4 <= resident_blocks() * 3 && width >= 128) {  // (the capacity is an upper bound)
      a.n_tiles = (int)((width + 127) / 128);
      static PerDeviceOnce narrow_configured;
      if (narrow_configured.needed()) {
        if (int rc = set_lds(row_tiled_kernel<MODE, 2, GATHER, 4, SAVE_GU>, W_LDS_BYTES)) return rc;
        narrow_configured.done();
      }
      const unsigned blocks = std::min(round8(tile_capacity * a.n_tiles), resident_blocks());
      hipLaunchKernelGGL((row_tiled_kernel<MODE, 2, GATHER, 4, SAVE_GU>), dim3(blocks), dim3(NT), W_LDS_BYTES, s, a);
      return check_launch(what);
    }
  }
  static PerDeviceOnce configured;  // one per kernel instantiation
  if (configured.needed()) {
    if (int rc = set_lds(row_tiled_kernel<MODE, 4, GATHER, 4, SAVE_GU>, W_LDS_BYTES)) return rc;
    configured.done();
  }
  const unsigned blocks = std::min(round8(tile_capacity * a.n_tiles), resident_blocks());
  hipLaunchKernelGGL((row_tiled_kernel<MODE, 4, GATHER, 4, SAVE_GU>), dim3(blocks), dim3(NT), W_LDS_BYTES, s, a);
  return check_launch(what);
}

int bf16_grouped_fwd(const void* rows, const int32_t* token_of_row, int64_t num_tokens, const void* w1,
                     const void* w3, const void* w2, const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* gate, void* up, void* h, void* y, int64_t D,
                     int64_t F, int stages, hipStream_t s) {
  RowArgs a{};
  a.seg_offsets = seg_offsets; a.seg_counts = seg_counts; a.tile_expert = tile_expert;
  a.tile_row0 = tile_row0; a.num_tiles = num_tiles; a.D = (int)D; a.F = (int)F;
  if (stages & STAGE_GATEUP) {
    a.a0 = (const uint16_t*)rows; a.a_src = token_of_row; a.a_rows = (int)num_tokens;
    a.b0 = (const uint16_t*)w1; a.b1 = (const uint16_t*)w3;
    a.o0 = (uint16_t*)gate; a.o1 = (uint16_t*)up; a.o2 = (uint16_t*)h;
    // gate == up == null: a forward-only caller; the kernel then writes h alone
    const bool save = gate != nullptr;
    int rc;
    if (token_of_row)
      rc = save ? launch_row<RM_GATEUP, true>(a, F, tile_capacity, s, "grouped gate/up")
                : launch_row<RM_GATEUP, true, false>(a, F, tile_capacity, s, "grouped gate/up (h only)");
    else
      rc = save ? launch_row<RM_GATEUP>(a, F, tile_capacity, s, "grouped gate/up")
                : launch_row<RM_GATEUP, false, false>(a, F, tile_capacity, s, "grouped gate/up (h only)");
    if (rc) return rc;
  }
  if (stages & STAGE_DOWN) {
    RowArgs b = a;
    b.a_src = nullptr;
    b.a0 = (const uint16_t*)h; b.b0 = (const uint16_t*)w2; b.o0 = (uint16_t*)y;
    if (int rc = launch_row<RM_DOWN>(b, D, tile_capacity, s, "grouped down")) return rc;
  }
  return MI355_OK;
}

// dx = dy . w[e] over the listed segments: dy (rows, O), w (El, O, I), dx (rows, I)
int bf16_grouped_linear_dx(const void* dy, const void* w, const int32_t* seg_offsets, const int32_t* seg_counts,
                           const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                           int64_t tile_capacity, void* dx, int64_t O, int64_t I, hipStream_t s) {
  RowArgs a{};
  a.seg_offsets = seg_offsets; a.seg_counts = seg_counts; a.tile_expert = tile_expert;
  a.tile_row0 = tile_row0; a.num_tiles = num_tiles; a.D = (int)O; a.F = (int)I;
  a.a0 = (const uint16_t*)dy; a.b0 = (const uint16_t*)w; a.o0 = (uint16_t*)dx;
  return launch_row<RM_DLIN>(a, I, tile_capacity, s, "grouped linear dx");
}

int bf16_fused_dot_slots(int64_t F) {
  // one partial per 128 output columns of the dH tile (two waves across its 256 columns)
  return (int)((F + 255) / 256) * 2;
}

// row_scale != null: the combine's backward is folded in.  dy is then the layer's output
// gradient (T, D), read through token_of_row and scaled by row_scale; `h` is written (it
// receives row_scale * h, the operand of dW2) and dot_partial gets the score-gradient pieces.
int bf16_grouped_bwd(const void* dy, const void* rows, const int32_t* token_of_row, int64_t num_tokens,
                     const void* w1, const void* w3, const void* w2, const void* gate, const void* up,
                     const void* h, const float* row_scale, float* dot_partial,
                     const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* dgate, void* dup, void* drows, void* dw1,
                     void* dw3, void* dw2, int64_t El, int64_t D, int64_t F, int stages,
                     hipStream_t s) {
  RowArgs a{};
  a.seg_offsets = seg_offsets; a.seg_counts = seg_counts; a.tile_expert = tile_expert;
  a.tile_row0 = tile_row0; a.num_tiles = num_tiles; a.D = (int)D; a.F = (int)F;
  if (stages & STAGE_DH) {
    a.a0 = (const uint16_t*)dy; a.b0 = (const uint16_t*)w2;
    a.gate = (const uint16_t*)gate; a.up = (const uint16_t*)up;
    a.o0 = (uint16_t*)dgate; a.o1 = (uint16_t*)dup;
    if (row_scale) {
      a.a_src = token_of_row; a.a_rows = (int)num_tokens; a.row_scale = row_scale; a.dot_partial = dot_partial;
      a.o2 = (uint16_t*)const_cast<void*>(h);
      a.dot_slots = bf16_fused_dot_slots(F);
      if (int rc = launch_row<RM_DH, true>(a, F, tile_capacity, s, "grouped dh + combine")) return rc;
      a.a_src = nullptr;
    } else {
      if (int rc = launch_row<RM_DH>(a, F, tile_capacity, s, "grouped dh")) return rc;
    }
  }
  if (drows && (stages & STAGE_DX)) {
    RowArgs b = a;
    b.a0 = (const uint16_t*)dgate; b.a1 = (const uint16_t*)dup;
    b.b0 = (const uint16_t*)w1; b.b1 = (const uint16_t*)w3; b.o0 = (uint16_t*)drows;
    if (int rc = launch_row<RM_DX>(b, D, tile_capacity, s, "grouped drows")) return rc;
  }
  static PerDeviceOnce wconfigured;
  if (wconfigured.needed()) {
    if (int rc = set_lds(wgrad_kernel<false>, W_LDS_BYTES)) return rc;
    if (int rc = set_lds(wgrad_kernel<true>, W_LDS_BYTES)) return rc;
    if (int rc = set_lds(wgrad_kernel<false, true>, W_LDS_BYTES)) return rc;
    wconfigured.done();
  }
  auto wgrad = [&](const void* A, const void* B, const int32_t* b_src, void* C, int64_t M, int64_t N, const char* what,
                   const int32_t* a_src = nullptr) {
    WgradArgs w{};
    w.a = (const uint16_t*)A; w.b = (const uint16_t*)B; w.c = (uint16_t*)C; w.b_src = b_src; w.a_src = a_src;
    w.src_rows = (int)num_tokens;
    w.seg_offsets = seg_offsets; w.seg_counts = seg_counts; w.El = (int)El; w.M = (int)M; w.N = (int)N;
    w.m_tiles = (int)((M + WBM - 1) / WBM); w.n_tiles = (int)((N + WBN - 1) / WBN);
    w.total = (int)(El * w.m_tiles * w.n_tiles);
    const dim3 grid(std::min(round8(w.total), resident_blocks()));
    if (a_src)
      hipLaunchKernelGGL((wgrad_kernel<false, true>), grid, dim3(NT), W_LDS_BYTES, s, w);
    else if (b_src)
      hipLaunchKernelGGL(wgrad_kernel<true>, grid, dim3(NT), W_LDS_BYTES, s, w);
    else
      hipLaunchKernelGGL(wgrad_kernel<false>, grid, dim3(NT), W_LDS_BYTES, s, w);
    return check_launch(what);
  };
  // folded combine: dW2 = (gathered output gradient)^T . (row_scale * h)
  if (dw2 && (stages & STAGE_DW2))
    if (int rc = wgrad(dy, h, nullptr, dw2, D, F, "grouped dw2", row_scale ? token_of_row : nullptr)) return rc;
  if (dw1 && (stages & STAGE_DW1)) if (int rc = wgrad(dgate, rows, token_of_row, dw1, F, D, "grouped dw1")) return rc;
  if (dw3 && (stages & STAGE_DW3)) if (int rc = wgrad(dup, rows, token_of_row, dw3, F, D, "grouped dw3")) return rc;
  return MI355_OK;
}

}  // namespace mi355
