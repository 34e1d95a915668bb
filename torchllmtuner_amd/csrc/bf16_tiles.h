// bf16 MFMA tile helpers shared by the grouped expert GEMMs and the router projections:
// vector types, the two LDS operand layouts and their fragment reads, and a barrier that
// leaves global memory traffic in flight.
//
// LDS layouts (no padding, XOR swizzles; 16-byte chunks), BK = 64 contraction elements
// per K step:
//   KC  contraction axis contiguous in HBM: [row][64 k], chunk c of row r stored at
//       c ^ ((r >> 1) & 7); a fragment is one ds_read_b128 (measured conflict-free;
//       the key r & 7 costs a 2-way conflict).
//   KS  contraction axis strided in HBM: [k][cols], chunk c of row k stored at
//       c ^ ((k & 3) << 2) (16 chunks or more per row); a fragment is two ds_read_b64_tr_b16 (LDS transpose
//       reads: lane i of a 16-lane group supplies the address of row i/4, 8-byte
//       piece i%4, and receives column i of the four rows).
// v_mfma_f32_32x32x16_bf16 takes per lane 8 bf16 of each operand (row lane%32,
// k = 8*(lane/32)..+7) and yields 16 fp32 (column lane%32, rows 8*(i/4) + 4*(lane/32) + i%4).
#pragma once
#include "common.h"

namespace mi355 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef short s16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x2 __attribute__((ext_vector_type(2)));

constexpr int BK = 64;

// KS swizzle key of LDS row k, in 16-byte chunks: a transpose read touches four
// consecutive k rows and 64 bytes of each per 32 lanes, and rows are a multiple of
// 256 bytes apart, so each row's four chunks are moved to their own quarter of the banks.
__device__ __forceinline__ int ks_key(int k) { return (k & 3) << 2; }

#define LDS_PTR(p) ((__attribute__((address_space(3))) s16x4*)(p))

// ---- fragment reads -----------------------------------------------------------------
__device__ __forceinline__ bf16x8 frag_kc(const uint16_t* tile, int row, int kk, int lane) {
  const int r = row + (lane & 31);
  const int c = kk * 2 + (lane >> 5);
  return *reinterpret_cast<const bf16x8*>(tile + r * BK + ((c ^ ((r >> 1) & 7)) << 3));
}

template <int COLS>
__device__ __forceinline__ bf16x8 frag_ks(const uint16_t* tile, int col, int kk, int lane) {
  const int g = lane >> 4, i = lane & 15;
  const int k = kk * 16 + 8 * (g >> 1) + (i >> 2);  // k & 3 == i >> 2 for both reads
  const int c = col + 16 * (g & 1) + 4 * (i & 3);
  const int off = (((c >> 3) ^ ks_key(k)) << 3) + (c & 7);
  const uint16_t* p = tile + k * COLS + off;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p + 4 * COLS));
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// ---- fragments for v_mfma_f32_16x16x32_bf16 -------------------------------------------
// Per lane 8 bf16 of each operand: row lane%16, k = 8*(lane/16)..+7 of a 32-wide K block;
// 4 fp32 of the result: column lane%16, rows 4*(lane/16) + i.  With random operand bits
// this shape sustains about 14 % more than 32x32x16 on MI355X (a quarter of the
// accumulator bytes per instruction for half the flops, and power is what limits both).
__device__ __forceinline__ bf16x8 frag16_kc(const uint16_t* tile, int row, int kk32, int lane) {
  const int r = row + (lane & 15);
  const int c = kk32 * 4 + (lane >> 4);
  return *reinterpret_cast<const bf16x8*>(tile + r * BK + ((c ^ ((r >> 1) & 7)) << 3));
}

// KS key for the 16x16x32 reader: 32 lanes of a transpose read touch rows k..k+3 and
// k+8..k+11, 32 bytes of each, so the eight rows get an eighth of the banks each.
__device__ __forceinline__ int ks_key16(int k) { return ((k & 3) << 2) | (((k >> 3) & 1) << 1); }

template <int COLS>
__device__ __forceinline__ bf16x8 frag16_ks(const uint16_t* tile, int col, int kk32, int lane) {
  const int g = lane >> 4, i = lane & 15;
  const int k = kk32 * 32 + 8 * g + (i >> 2);  // key of row k + 4 equals that of row k
  const int c = col + 4 * (i & 3);
  const int off = (((c >> 3) ^ ks_key16(k)) << 3) + (c & 7);
  const uint16_t* p = tile + k * COLS + off;
  const s16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p));
  const s16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16(LDS_PTR(p + 4 * COLS));
  const s16x8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return __builtin_bit_cast(bf16x8, v);
}

// Workgroup barrier that waits for this wave's own LDS operations only: global loads and
// stores stay in flight across it.
__device__ __forceinline__ void phase_barrier() {
  __builtin_amdgcn_sched_barrier(0);
  __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
  __builtin_amdgcn_s_barrier();
  __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ uint32_t pack2(float a, float b) { return pack_bf16x2(a, b); }

// ---- epilogue staging -----------------------------------------------------------------
// A wave parks its 64 x W sub-tile (bf16) in its private LDS region, [64][W + 8], then
// streams it out as 16-byte row pieces.  acc was produced with the weight fragment as
// the first MFMA operand: lane = output row (lane & 31), registers = output columns.
template <int W>
struct WaveStage {
  static constexpr int PITCH = W + 8;
  static constexpr int ELEMS = 64 * PITCH;
  // element (row m of 64, col n of W) for register i of the accumulator tile (mi, nj-th 32 columns)
  __device__ static __forceinline__ void put4(uint16_t* st, int mi, int col0, int lane, int q,
                                              float v0, float v1, float v2, float v3) {
    const int m = mi * 32 + (lane & 31);
    const int n = col0 + q * 8 + (lane >> 5) * 4;
    u32x2 pk = {pack2(v0, v1), pack2(v2, v3)};
    *reinterpret_cast<u32x2*>(st + m * PITCH + n) = pk;
  }
  // the same for a 16 x 16 accumulator tile (mi-th 16 rows): lane = row lane & 15,
  // registers = columns col0 + 4 * (lane >> 4) .. + 3
  __device__ static __forceinline__ void put16(uint16_t* st, int mi, int col0, int lane, float v0, float v1,
                                               float v2, float v3) {
    const int m = mi * 16 + (lane & 15);
    const int n = col0 + 4 * (lane >> 4);
    u32x2 pk = {pack2(v0, v1), pack2(v2, v3)};
    *reinterpret_cast<u32x2*>(st + m * PITCH + n) = pk;
  }
};

}  // namespace mi355
