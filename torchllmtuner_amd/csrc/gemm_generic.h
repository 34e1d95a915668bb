// Generic strided GEMM with fp32 MFMA accumulation (v_mfma_f32_32x32x2_f32).
//
// C(m,n) = sum_k A(m,k) * B(k,n) with arbitrary element strides on A and B, any
// mix of fp32 / bf16 storage, and three ways of slicing the problem:
//   DENSE   one problem, optional split-K into fp32 partials
//   ROWSEG  the M axis is a list of expert segments (tile list); B is picked per
//           expert (forward and data-gradient grouped GEMMs)
//   KSEG    one problem per expert whose K range is that expert's row segment
//           (weight-gradient grouped GEMMs)
// It carries the fp32 configuration, the router projections and every shape the
// bf16 MFMA kernels do not accept; it is not the bf16 hot path.
#pragma once

#include "common.h"

namespace mi355 {

enum GemmMode { GEMM_DENSE = 0, GEMM_ROWSEG = 1, GEMM_KSEG = 2 };

struct GemmArgs {
  const void* A;
  const void* B;
  void* C;
  const float* bias;  // per output column, fp32, may be null
  int64_t a_rs, a_cs; // A(m,k) = A[m*a_rs + k*a_cs]
  int64_t b_rs, b_cs; // B(k,n) = B[k*b_rs + n*b_cs]
  int64_t ldc;
  int64_t b_es, c_es; // expert strides (elements) for ROWSEG (B) and KSEG (C)
  int M, N, K;
  int mode;
  int accumulate;     // C += result (read-modify-write in C's dtype)
  int ksplit;         // DENSE only: >1 writes fp32 partials to C + z*M*ldc
  int tile_m;         // ROWSEG: rows per listed tile (multiple of 64)
  const int32_t* seg_offsets;
  const int32_t* seg_counts;
  const int32_t* tile_expert;
  const int32_t* tile_row0;
  const int32_t* num_tiles;
};

// a_dtype / b_dtype / c_dtype are MI355_F32 or MI355_BF16.
int launch_gemm(const GemmArgs& args, int a_dtype, int b_dtype, int c_dtype,
                dim3 grid, hipStream_t stream);

// Grid helpers.
dim3 gemm_grid_dense(int M, int N, int ksplit);
dim3 gemm_grid_rowseg(int64_t tile_capacity, int tile_m, int N);
dim3 gemm_grid_kseg(int M, int N, int El);

// out = sum_z partial[z] (+bias), partial: (ksplit, M, N) fp32 contiguous.
int launch_splitk_reduce(const float* partial, void* out, int out_dtype, int64_t MN,
                         int ksplit, hipStream_t stream);

// Router projections as three bf16 MFMAs per fp32 product (router_gemm.hip): bf16 tokens,
// fp32 weights, D and E multiples of 64.
bool router_x3_ok(int x_dtype, int w_dtype, int64_t D, int64_t E);
int64_t router_x3_fwd_workspace(int64_t T, int64_t D, int64_t E);
int64_t router_x3_bwd_workspace(int64_t T, int64_t D, int64_t E);
int router_x3_fwd(const void* x, const float* w, const float* bias, float* logits, void* workspace,
                  int64_t T, int64_t D, int64_t E, hipStream_t s);
int router_x3_bwd(const float* dlogits, const void* x, const float* w, void* dx, float* dw,
                  void* workspace, int64_t T, int64_t D, int64_t E, hipStream_t s);

}  // namespace mi355
