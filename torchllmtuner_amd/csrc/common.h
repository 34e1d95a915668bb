// Shared helpers for the gfx950 MoE kernels: error reporting, bf16 conversion,
// wave-level reductions.  Internal to the library; the public surface is
// include/mi355_moe.h.
#pragma once

#include <hip/hip_runtime.h>

#include <atomic>
#include <stdint.h>

#include <cstdarg>
#include <cstdio>

#include "../../include/mi355_moe.h"

namespace mi355 {

constexpr int kWave = 64;

// ---- error text (thread-local) ---------------------------------------------
char* error_buffer();
int fail(int code, const char* fmt, ...);
int check_launch(const char* what);

#define MI355_REQUIRE(cond, ...)                         \
  do {                                                   \
    if (!(cond)) return mi355::fail(MI355_EINVAL, __VA_ARGS__); \
  } while (0)

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }

// One-time set-up per device (kernel attributes are per device): `needed()` is true until
// `done()` has been called with the same device current.  Safe to race: set-up is idempotent.
class PerDeviceOnce {
 public:
  bool needed() const { return !(mask_.load(std::memory_order_acquire) & bit()); }
  void done() { mask_.fetch_or(bit(), std::memory_order_release); }

 private:
  static uint64_t bit() {
    int dev = 0;
    (void)hipGetDevice(&dev);
    return 1ull << (dev & 63);
  }
  std::atomic<uint64_t> mask_{0};
};

// ---- bf16 <-> f32, round to nearest even (what torch's .to(bfloat16) does) ----
__device__ __forceinline__ float bf16_to_f32(uint16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}
// gfx950 converts in hardware (v_cvt_pk_bf16_f32, round to nearest even, NaN stays NaN).
typedef __bf16 mi355_bf16x2 __attribute__((ext_vector_type(2)));
typedef float mi355_f32x2 __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
}
// {lo, hi} -> one dword holding bf16(lo) | bf16(hi) << 16
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  const mi355_f32x2 v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, mi355_bf16x2));
}
__device__ __forceinline__ float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

// Height of the row tiles of a segment of `count` rows: its ceil(count / tile_m) tiles are made
// equally tall (to a multiple of the 16-row MFMA block) instead of tile_m, tile_m, ..., rest.
// A rest of a few rows costs most of a full tile (its weight tile is staged all the same) and
// runs out of step with its neighbours, which then miss each other's operands in L2; equal
// tiles cost their share of the rows and stay in step.  Never more than tile_m, never leaves
// a tile empty.  The plan kernels and every kernel that walks the tile list use this one rule.
__host__ __device__ inline int even_tile_rows(int count, int tile_m) {
  const int nt = (count + tile_m - 1) / tile_m;
  if (nt <= 1) return tile_m;
  const int per = (count + nt - 1) / nt;
  return (per + 15) / 16 * 16;
}

// 16-byte load of data that is read once and not again soon (a row stream larger than the
// caches): the non-temporal hint keeps it from displacing what other loads reuse.  Measured on
// the row gathers here, beyond the size the caches hold: 5.1 -> 6.0 TB/s.
__device__ __forceinline__ uint4 load_stream(const uint4* p) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t v = __builtin_nontemporal_load(reinterpret_cast<const u32x4_t*>(p));
  return make_uint4(v[0], v[1], v[2], v[3]);
}

// the same for a 16-byte store of data that is written once, in a stream larger than the caches
__device__ __forceinline__ void store_stream(uint4* p, const uint4& v) {
  typedef uint32_t u32x4_t __attribute__((ext_vector_type(4)));
  const u32x4_t w = {v.x, v.y, v.z, v.w};
  __builtin_nontemporal_store(w, reinterpret_cast<u32x4_t*>(p));
}

template <typename T>
__device__ __forceinline__ float load_as_f32(const T* p);
template <>
__device__ __forceinline__ float load_as_f32<float>(const float* p) { return *p; }
template <>
__device__ __forceinline__ float load_as_f32<uint16_t>(const uint16_t* p) { return bf16_to_f32(*p); }
// fp64 storage read by a kernel that computes in fp32 (the router: `.float()` of its operands)
template <>
__device__ __forceinline__ float load_as_f32<double>(const double* p) { return static_cast<float>(*p); }

template <typename T>
__device__ __forceinline__ void store_from_f32(T* p, float v);
template <>
__device__ __forceinline__ void store_from_f32<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_from_f32<uint16_t>(uint16_t* p, float v) { *p = f32_to_bf16(v); }
template <>
__device__ __forceinline__ void store_from_f32<double>(double* p, float v) { *p = static_cast<double>(v); }

// ---- wave reductions ---------------------------------------------------------
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, kWave);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, kWave));
  return v;
}

__device__ __forceinline__ float silu_f32(float g) { return g / (1.0f + __expf(-g)); }

}  // namespace mi355
