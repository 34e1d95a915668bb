// Measurement probe, used by the benchmark only (not part of the MoE C ABI): what the
// matrix cores of this card sustain on the two instructions the grouped GEMMs use, with
// operands held in registers, so that a kernel's rate can be set against the rate the
// silicon holds under its own power management rather than against the data-sheet
// figure alone.  Random operand bits draw markedly more power than constant ones, and
// the sustained clock follows; both cases are offered.
#include <hip/hip_runtime.h>

#include <cstdint>

namespace {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t mix(uint32_t x) {
  x ^= x >> 16; x *= 0x7feb352du; x ^= x >> 15; x *= 0x846ca68bu; x ^= x >> 16;
  return x;
}

// 8 waves per workgroup, each wave a 64 x 128 accumulator tile (2 x 4 MFMA tiles), the
// shape of the grouped GEMM main loop.  clocks[2*b] = core cycles, clocks[2*b+1] = 100 MHz
// ticks spent by block b.
__global__ __launch_bounds__(512, 2) void probe_mfma_kernel(float* sink, unsigned long long* clocks,
                                                           int iters, int random_bits) {
  const uint32_t seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u;
  bf16x8 a[2], b[4];
#pragma unroll
  for (int i = 0; i < 6; ++i) {
    u32x4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      // two bf16 per dword around 1.0: exponent fixed, sign and mantissa random or constant
      const uint32_t r = random_bits ? mix(seed + i * 97u + w * 7919u) : 0u;
      v[w] = 0x3f803f80u ^ (r & 0x807f807fu);
    }
    if (i < 2) a[i] = __builtin_bit_cast(bf16x8, v); else b[i - 2] = __builtin_bit_cast(bf16x8, v);
  }
  f32x16 acc[2][4];
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) acc[m][n][i] = 0.0f;
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int n = 0; n < 4; ++n)
        acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b[n], a[m], acc[m][n], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.0f;
#pragma unroll
  for (int m = 0; m < 2; ++m)
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 16; ++i) s += acc[m][n][i];
  if (s == 1234.5f) sink[0] = s;  // keeps the loop alive
  if (threadIdx.x == 0 && clocks) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

// The same per-wave tile as 4 x 8 tiles of v_mfma_f32_16x16x32_bf16 (the shape of the
// row-tiled grouped GEMMs); one iteration is 32 instructions of 16384 flops.
__global__ __launch_bounds__(512, 2) void probe_mfma16_kernel(float* sink, unsigned long long* clocks,
                                                             int iters, int random_bits) {
  const uint32_t seed = threadIdx.x * 2654435761u + blockIdx.x * 40503u;
  bf16x8 a[4], b[8];
#pragma unroll
  for (int i = 0; i < 12; ++i) {
    u32x4 v;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const uint32_t r = random_bits ? mix(seed + i * 97u + w * 7919u) : 0u;
      v[w] = 0x3f803f80u ^ (r & 0x807f807fu);
    }
    if (i < 4) a[i] = __builtin_bit_cast(bf16x8, v); else b[i - 4] = __builtin_bit_cast(bf16x8, v);
  }
  typedef float f32x4 __attribute__((ext_vector_type(4)));
  f32x4 acc[4][8];
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[m][n][i] = 0.0f;
  const unsigned long long c0 = clock64(), w0 = wall_clock64();
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
      for (int n = 0; n < 8; ++n)
        acc[m][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(b[n], a[m], acc[m][n], 0, 0, 0);
  }
  const unsigned long long c1 = clock64(), w1 = wall_clock64();
  float s = 0.0f;
#pragma unroll
  for (int m = 0; m < 4; ++m)
#pragma unroll
    for (int n = 0; n < 8; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) s += acc[m][n][i];
  if (s == 1234.5f) sink[0] = s;
  if (threadIdx.x == 0 && clocks) {
    clocks[2 * blockIdx.x] = c1 - c0;
    clocks[2 * blockIdx.x + 1] = w1 - w0;
  }
}

}  // namespace

// Launches `blocks` workgroups of the probe on `stream`.  shape 0: 32x32x16, one iteration =
// 8 instructions of 32768 flops; shape 1: 16x16x32, one iteration = 32 instructions of
// 16384 flops; either way flops = blocks * 8 waves * iters * 262144 * (shape + 1).
// `clocks` (2 * blocks uint64, device) may be null.
extern "C" int mi355_probe_mfma(float* sink, unsigned long long* clocks, int blocks, int iters,
                                int random_bits, int shape, void* stream) {
  if (!sink || blocks < 1 || iters < 1 || shape < 0 || shape > 1) return -1;
  if (shape == 0)
    hipLaunchKernelGGL(probe_mfma_kernel, dim3(blocks), dim3(512), 0, static_cast<hipStream_t>(stream), sink,
                       clocks, iters, random_bits);
  else
    hipLaunchKernelGGL(probe_mfma16_kernel, dim3(blocks), dim3(512), 0, static_cast<hipStream_t>(stream), sink,
                       clocks, iters, random_bits);
  return hipGetLastError() == hipSuccess ? 0 : -2;
}
