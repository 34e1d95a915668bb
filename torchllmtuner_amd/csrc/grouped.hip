// Grouped SwiGLU experts: C entry points and the generic (any dtype, any shape)
// path.  bf16 problems whose D and F are multiples of 64 go to the MFMA kernels of
// grouped_bf16.hip; everything else (fp32, fp64, odd shapes) runs the strided GEMM of
// gemm_generic.hip (fp32 MFMA; fp64 MFMA for fp64) plus two small elementwise kernels.
#include <cstdlib>

#include "common.h"
#include "gemm_generic.h"

namespace mi355 {

bool bf16_fast_path_ok(int64_t D, int64_t F);
int bf16_row_tile_m();
// rows per entry of the plan's tile list: the row-tile height of the bf16 MFMA kernels, for
// every dtype (a plan is built from expert ids alone, before the dtype of its rows is known;
// the generic kernels walk tiles of any multiple of 64 rows)
inline int tile_m_for(int dtype) { (void)dtype; return bf16_row_tile_m(); }
int bf16_grouped_fwd(const void* rows, const int32_t* token_of_row, int64_t num_tokens, const void* w1,
                     const void* w3, const void* w2, const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* gate, void* up, void* h, void* y, int64_t D,
                     int64_t F, int stages, hipStream_t s);
int bf16_fused_dot_slots(int64_t F);
int bf16_grouped_linear_dx(const void* dy, const void* w, const int32_t* seg_offsets, const int32_t* seg_counts,
                           const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                           int64_t tile_capacity, void* dx, int64_t O, int64_t I, hipStream_t s);
int bf16_grouped_bwd(const void* dy, const void* rows, const int32_t* token_of_row, int64_t num_tokens,
                     const void* w1, const void* w3, const void* w2, const void* gate, const void* up,
                     const void* h, const float* row_scale, float* dot_partial,
                     const int32_t* seg_offsets, const int32_t* seg_counts,
                     const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
                     int64_t tile_capacity, void* dgate, void* dup, void* drows, void* dw1,
                     void* dw3, void* dw2, int64_t El, int64_t D, int64_t F, int stages,
                     hipStream_t s);

namespace {

template <typename T>
__device__ __forceinline__ float rnd(float v);
template <>
__device__ __forceinline__ float rnd<float>(float v) { return v; }
template <>
__device__ __forceinline__ float rnd<uint16_t>(float v) { return round_bf16(v); }

// h = silu(gate) * up over the first *total_rows rows, with the activation dtype's
// rounding after the SiLU and after the product.
template <typename T>
__global__ void swiglu_fwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                  T* __restrict__ h, const int32_t* __restrict__ total_rows, int F) {
  const int64_t n = static_cast<int64_t>(*total_rows) * F;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const float g = load_as_f32(gate + i);
    const float s = rnd<T>(g / (1.0f + expf(-g)));
    store_from_f32(h + i, s * load_as_f32(up + i));
  }
}

// in: dgate holds dh.  out: dgate = dh*up*silu'(gate), dup = dh*silu(gate).
template <typename T>
__global__ void swiglu_bwd_kernel(const T* __restrict__ gate, const T* __restrict__ up,
                                  T* __restrict__ dgate, T* __restrict__ dup,
                                  const int32_t* __restrict__ total_rows, int F) {
  const int64_t n = static_cast<int64_t>(*total_rows) * F;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const float dh = load_as_f32(dgate + i);
    const float g = load_as_f32(gate + i);
    const float u = load_as_f32(up + i);
    const float sig = 1.0f / (1.0f + expf(-g));
    const float s = rnd<T>(g * sig);
    const float ds = rnd<T>(dh * u);
    store_from_f32(dup + i, dh * s);
    store_from_f32(dgate + i, ds * (sig * (1.0f + g * (1.0f - sig))));
  }
}

// the same two in fp64, for fp64 experts (every step of the reference's fp64 path is fp64)
__global__ void swiglu_fwd_f64_kernel(const double* __restrict__ gate, const double* __restrict__ up,
                                      double* __restrict__ h, const int32_t* __restrict__ total_rows, int F) {
  const int64_t n = static_cast<int64_t>(*total_rows) * F;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const double g = gate[i];
    h[i] = g / (1.0 + exp(-g)) * up[i];
  }
}

__global__ void swiglu_bwd_f64_kernel(const double* __restrict__ gate, const double* __restrict__ up,
                                      double* __restrict__ dgate, double* __restrict__ dup,
                                      const int32_t* __restrict__ total_rows, int F) {
  const int64_t n = static_cast<int64_t>(*total_rows) * F;
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n;
       i += static_cast<int64_t>(gridDim.x) * blockDim.x) {
    const double dh = dgate[i], g = gate[i], u = up[i];
    const double sig = 1.0 / (1.0 + exp(-g));
    dup[i] = dh * (g * sig);
    dgate[i] = dh * u * (sig * (1.0 + g * (1.0 - sig)));
  }
}

struct Seg {
  const int32_t *seg_offsets, *seg_counts, *tile_expert, *tile_row0, *num_tiles;
  int64_t tile_capacity;
};

// C(rows, N) = A(rows, K) . B[e]  over the tile-listed rows
int rowseg(const Seg& sg, const void* A, int64_t lda, const void* B, int64_t b_rs, int64_t b_cs,
           int64_t b_es, void* C, int64_t N, int64_t K, int dtype, int accumulate, hipStream_t s) {
  GemmArgs g{};
  g.A = A; g.B = B; g.C = C;
  g.a_rs = lda; g.a_cs = 1; g.b_rs = b_rs; g.b_cs = b_cs; g.b_es = b_es;
  g.ldc = N; g.M = 0; g.N = (int)N; g.K = (int)K;
  g.mode = GEMM_ROWSEG; g.accumulate = accumulate; g.ksplit = 1; g.tile_m = tile_m_for(dtype);
  g.seg_offsets = sg.seg_offsets; g.seg_counts = sg.seg_counts; g.tile_expert = sg.tile_expert;
  g.tile_row0 = sg.tile_row0; g.num_tiles = sg.num_tiles;
  return launch_gemm(g, dtype, dtype, dtype, gemm_grid_rowseg(sg.tile_capacity, tile_m_for(dtype), (int)N), s);
}

// C[e](M, N) = sum_{r in segment e} A[r][m] * B[r][n]
int kseg(const Seg& sg, const void* A, const void* B, void* C, int64_t M, int64_t N, int64_t El,
         int dtype, hipStream_t s) {
  GemmArgs g{};
  g.A = A; g.B = B; g.C = C;
  g.a_rs = 1; g.a_cs = M; g.b_rs = N; g.b_cs = 1; g.c_es = M * N;
  g.ldc = N; g.M = (int)M; g.N = (int)N; g.K = 0;
  g.mode = GEMM_KSEG; g.ksplit = 1;
  g.seg_offsets = sg.seg_offsets; g.seg_counts = sg.seg_counts;
  return launch_gemm(g, dtype, dtype, dtype, gemm_grid_kseg((int)M, (int)N, (int)El), s);
}

int check_common(const char* who, int dtype, int64_t El, int64_t D, int64_t F, int64_t row_capacity,
                 int64_t tile_capacity) {
  MI355_REQUIRE(dtype == MI355_F32 || dtype == MI355_BF16 || dtype == MI355_F64, "%s: unknown dtype %d", who, dtype);
  MI355_REQUIRE(El >= 1 && D >= 1 && F >= 1, "%s: bad shape El=%lld D=%lld F=%lld", who, (long long)El,
                (long long)D, (long long)F);
  MI355_REQUIRE(D < (1ll << 24) && F < (1ll << 24) && D * F < (1ll << 31), "%s: D*F exceeds int32", who);
  MI355_REQUIRE(row_capacity >= 0 && row_capacity < (1ll << 31) && tile_capacity >= 0 &&
                    tile_capacity < (1ll << 24),
                "%s: bad capacity", who);
  return MI355_OK;
}

// The fused token gather reads rows[token_of_row[r]] with a 32-bit byte offset and clamps the
// index to [0, num_tokens): the token matrix must hold at least one row and stay below 4 GiB.
int check_gather(const char* who, const int32_t* token_of_row, int64_t num_tokens, int64_t D, int dtype) {
  if (!token_of_row) return MI355_OK;
  if (dtype != MI355_BF16) return fail(MI355_EUNSUP, "%s: the token gather exists for bf16 only", who);
  MI355_REQUIRE(num_tokens >= 1, "%s: token_of_row given but num_tokens = %lld", who, (long long)num_tokens);
  MI355_REQUIRE(num_tokens < (1ll << 31) && num_tokens * D * 2 < (1ll << 32),
                "%s: gathered token matrix of %lld x %lld bf16 exceeds the 4 GiB the fused gather addresses; "
                "materialise the rows with mi355_permute_rows_fwd instead",
                who, (long long)num_tokens, (long long)D);
  return MI355_OK;
}

}  // namespace
}  // namespace mi355

using namespace mi355;

extern "C" int64_t mi355_grouped_tile_m(int dtype) {
  return tile_m_for(dtype);
}

extern "C" int mi355_grouped_swiglu_fwd(const void* rows, const int32_t* token_of_row, int64_t num_tokens,
                                        const void* w1, const void* w3, const void* w2, int dtype, const int32_t* seg_offsets,
                                        const int32_t* seg_counts, const int32_t* tile_expert,
                                        const int32_t* tile_row0, const int32_t* num_tiles,
                                        int64_t tile_capacity, void* gate, void* up, void* h, void* y,
                                        int64_t El, int64_t D, int64_t F, int64_t row_capacity,
                                        void* stream) {
  if (int rc = check_common("grouped_swiglu_fwd", dtype, El, D, F, row_capacity, tile_capacity)) return rc;
  if (int rc = check_gather("grouped_swiglu_fwd", row_capacity > 0 ? token_of_row : nullptr, num_tokens, D, dtype)) return rc;
  if (row_capacity == 0 || tile_capacity == 0) return MI355_OK;
  MI355_REQUIRE(rows && w1 && w3 && w2 && seg_offsets && seg_counts && tile_expert && tile_row0 &&
                    num_tiles && h && y,
                "grouped_swiglu_fwd: null pointer");
  // gate and up may both be null (nobody will run the backward): the bf16 MFMA path then skips
  // those two output streams; the other paths use them as their own intermediates
  MI355_REQUIRE((gate == nullptr) == (up == nullptr), "grouped_swiglu_fwd: gate and up must be given or omitted together");
  const bool fast = dtype == MI355_BF16 && bf16_fast_path_ok(D, F);
  MI355_REQUIRE(gate != nullptr || fast,
                "grouped_swiglu_fwd: gate and up can only be omitted for bf16 with D and F multiples of 64 (>= 384)");
  hipStream_t s = as_stream(stream);
  if (fast)
    return bf16_grouped_fwd(rows, token_of_row, num_tokens, w1, w3, w2, seg_offsets, seg_counts, tile_expert,
                            tile_row0, num_tiles, tile_capacity, gate, up, h, y, D, F, 3, s);
  if (token_of_row)
    return fail(MI355_EUNSUP, "grouped_swiglu_fwd: the token gather needs bf16 with D and F multiples of 64; "
                              "materialise the rows with mi355_permute_rows_fwd instead");
  const Seg sg{seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity};
  // gate/up: B(k=d, n=f) = w[e][f][d]
  if (int rc = rowseg(sg, rows, D, w1, 1, D, F * D, gate, F, D, dtype, 0, s)) return rc;
  if (int rc = rowseg(sg, rows, D, w3, 1, D, F * D, up, F, D, dtype, 0, s)) return rc;
  const unsigned blocks = (unsigned)std::min<int64_t>((row_capacity * F + 255) / 256, 8192);
  if (dtype == MI355_F32)
    hipLaunchKernelGGL(swiglu_fwd_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gate,
                       (const float*)up, (float*)h, seg_offsets + El, (int)F);
  else if (dtype == MI355_F64)
    hipLaunchKernelGGL(swiglu_fwd_f64_kernel, dim3(blocks), dim3(256), 0, s, (const double*)gate,
                       (const double*)up, (double*)h, seg_offsets + El, (int)F);
  else
    hipLaunchKernelGGL(swiglu_fwd_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s,
                       (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)h, seg_offsets + El, (int)F);
  if (int rc = check_launch("swiglu_fwd")) return rc;
  // down: B(k=f, n=d) = w2[e][d][f]
  return rowseg(sg, h, F, w2, 1, F, D * F, y, D, F, dtype, 0, s);
}

extern "C" int mi355_grouped_swiglu_bwd(const void* dy, const void* rows,
                                        const int32_t* token_of_row, int64_t num_tokens, const void* w1,
                                        const void* w3, const void* w2, const void* gate,
                                        const void* up, const void* h, int dtype,
                                        const int32_t* seg_offsets, const int32_t* seg_counts,
                                        const int32_t* tile_expert, const int32_t* tile_row0,
                                        const int32_t* num_tiles, int64_t tile_capacity, void* dgate,
                                        void* dup, void* drows, void* dw1, void* dw3, void* dw2,
                                        int64_t El, int64_t D, int64_t F, int64_t row_capacity,
                                        void* stream) {
  if (int rc = check_common("grouped_swiglu_bwd", dtype, El, D, F, row_capacity, tile_capacity)) return rc;
  if (int rc = check_gather("grouped_swiglu_bwd", row_capacity > 0 && tile_capacity > 0 ? token_of_row : nullptr,
                            num_tokens, D, dtype))
    return rc;
  MI355_REQUIRE(seg_offsets && seg_counts && num_tiles, "grouped_swiglu_bwd: null plan pointer");
  MI355_REQUIRE(row_capacity == 0 || (dy && rows && w1 && w3 && w2 && gate && up && h && dgate && dup &&
                                      tile_expert && tile_row0),
                "grouped_swiglu_bwd: null pointer");
  hipStream_t s = as_stream(stream);
  if (dtype == MI355_BF16 && bf16_fast_path_ok(D, F) && row_capacity > 0 && tile_capacity > 0)
    return bf16_grouped_bwd(
        dy, rows, token_of_row, num_tokens, w1, w3, w2, gate, up, h, nullptr, nullptr, seg_offsets, seg_counts,
        tile_expert, tile_row0, num_tiles, tile_capacity, dgate, dup, drows, dw1, dw3, dw2, El, D, F, 0x7c, s);
  // (with no rows at all nothing is gathered: only the zero weight gradients remain to be written)
  if (token_of_row && row_capacity > 0 && tile_capacity > 0)
    return fail(MI355_EUNSUP, "grouped_swiglu_bwd: the token gather needs bf16 with D and F multiples of 64");
  const Seg sg{seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity};
  if (row_capacity > 0 && tile_capacity > 0) {
    // dh = dy . w2[e]: B(k=d, n=f) = w2[e][d][f]   (lands in dgate, rewritten in place below)
    if (int rc = rowseg(sg, dy, D, w2, F, 1, D * F, dgate, F, D, dtype, 0, s)) return rc;
    const unsigned blocks = (unsigned)std::min<int64_t>((row_capacity * F + 255) / 256, 8192);
    if (dtype == MI355_F32)
      hipLaunchKernelGGL(swiglu_bwd_kernel<float>, dim3(blocks), dim3(256), 0, s, (const float*)gate,
                         (const float*)up, (float*)dgate, (float*)dup, seg_offsets + El, (int)F);
    else if (dtype == MI355_F64)
      hipLaunchKernelGGL(swiglu_bwd_f64_kernel, dim3(blocks), dim3(256), 0, s, (const double*)gate,
                         (const double*)up, (double*)dgate, (double*)dup, seg_offsets + El, (int)F);
    else
      hipLaunchKernelGGL(swiglu_bwd_kernel<uint16_t>, dim3(blocks), dim3(256), 0, s,
                         (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)dgate, (uint16_t*)dup,
                         seg_offsets + El, (int)F);
    if (int rc = check_launch("swiglu_bwd")) return rc;
    if (drows) {
      // drows = dgate . w1[e] + dup . w3[e]: B(k=f, n=d) = w[e][f][d]
      if (int rc = rowseg(sg, dgate, F, w1, D, 1, F * D, drows, D, F, dtype, 0, s)) return rc;
      if (int rc = rowseg(sg, dup, F, w3, D, 1, F * D, drows, D, F, dtype, 1, s)) return rc;
    }
  }
  // weight gradients also cover the no-rows case: every expert's gradient is written (zeros)
  if (dw2) if (int rc = kseg(sg, dy, h, dw2, D, F, El, dtype, s)) return rc;
  if (dw1) if (int rc = kseg(sg, dgate, rows, dw1, F, D, El, dtype, s)) return rc;
  if (dw3) if (int rc = kseg(sg, dup, rows, dw3, F, D, El, dtype, s)) return rc;
  return MI355_OK;
}

extern "C" int mi355_grouped_swiglu_stage(int stage, const void* dy, const void* rows,
                                          const int32_t* token_of_row, int64_t num_tokens, const void* w1, const void* w3, const void* w2, void* gate, void* up,
                                          void* h, void* y, const int32_t* seg_offsets,
                                          const int32_t* seg_counts, const int32_t* tile_expert,
                                          const int32_t* tile_row0, const int32_t* num_tiles,
                                          int64_t tile_capacity, void* dgate, void* dup, void* drows,
                                          void* dw1, void* dw3, void* dw2, int64_t El, int64_t D,
                                          int64_t F, int64_t row_capacity, void* stream) {
  if (int rc = check_common("grouped_swiglu_stage", MI355_BF16, El, D, F, row_capacity, tile_capacity)) return rc;
  MI355_REQUIRE(bf16_fast_path_ok(D, F), "grouped_swiglu_stage: needs bf16 with D and F multiples of 64");
  MI355_REQUIRE(stage > 0 && stage < 128 && (stage & (stage - 1)) == 0, "grouped_swiglu_stage: one stage bit expected");
  if (row_capacity == 0 || tile_capacity == 0) return MI355_OK;
  if (int rc = check_gather("grouped_swiglu_stage", token_of_row, num_tokens, D, MI355_BF16)) return rc;
  hipStream_t s = as_stream(stream);
  if (stage <= 2)
    return bf16_grouped_fwd(rows, token_of_row, num_tokens, w1, w3, w2, seg_offsets, seg_counts, tile_expert,
                            tile_row0, num_tiles, tile_capacity, gate, up, h, y, D, F, stage, s);
  return bf16_grouped_bwd(
      dy, rows, token_of_row, num_tokens, w1, w3, w2, gate, up, h, nullptr, nullptr, seg_offsets, seg_counts,
      tile_expert, tile_row0, num_tiles, tile_capacity, dgate, dup, drows, dw1, dw3, dw2, El, D, F, stage, s);
}

// ---- one grouped linear map: y[r] = x[r] . w[e(r)]^T (the reference's GroupedExperts._grouped_mm) ----
extern "C" int mi355_grouped_linear_fwd(const void* x, const void* w, int dtype, const int32_t* seg_offsets,
                                        const int32_t* seg_counts, const int32_t* tile_expert,
                                        const int32_t* tile_row0, const int32_t* num_tiles, int64_t tile_capacity,
                                        void* y, int64_t El, int64_t I, int64_t O, int64_t row_capacity,
                                        void* stream) {
  if (int rc = check_common("grouped_linear_fwd", dtype, El, O, I, row_capacity, tile_capacity)) return rc;
  if (row_capacity == 0 || tile_capacity == 0) return MI355_OK;
  MI355_REQUIRE(x && w && y && seg_offsets && seg_counts && tile_expert && tile_row0 && num_tiles,
                "grouped_linear_fwd: null pointer");
  hipStream_t s = as_stream(stream);
  if (dtype == MI355_BF16 && bf16_fast_path_ok(O, I))
    // the down projection's kernel is this product: rows (R, I) . w[e] (O, I)^T
    return bf16_grouped_fwd(nullptr, nullptr, 0, nullptr, nullptr, w, seg_offsets, seg_counts, tile_expert, tile_row0,
                            num_tiles, tile_capacity, nullptr, nullptr, const_cast<void*>(x), y, O, I, 2, s);
  const Seg sg{seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity};
  // B(k=i, n=o) = w[e][o][i]
  return rowseg(sg, x, I, w, 1, I, O * I, y, O, I, dtype, 0, s);
}

extern "C" int mi355_grouped_linear_bwd(const void* dy, const void* x, const void* w, int dtype,
                                        const int32_t* seg_offsets, const int32_t* seg_counts,
                                        const int32_t* tile_expert, const int32_t* tile_row0,
                                        const int32_t* num_tiles, int64_t tile_capacity, void* dx, void* dw,
                                        int64_t El, int64_t I, int64_t O, int64_t row_capacity, void* stream) {
  if (int rc = check_common("grouped_linear_bwd", dtype, El, O, I, row_capacity, tile_capacity)) return rc;
  MI355_REQUIRE(seg_offsets && seg_counts && num_tiles, "grouped_linear_bwd: null plan pointer");
  const bool rows = row_capacity > 0 && tile_capacity > 0;
  MI355_REQUIRE(!rows || (dy && x && w && tile_expert && tile_row0), "grouped_linear_bwd: null pointer");
  hipStream_t s = as_stream(stream);
  const Seg sg{seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity};
  if (dtype == MI355_BF16 && bf16_fast_path_ok(O, I) && rows) {
    if (dx)
      if (int rc = bf16_grouped_linear_dx(dy, w, seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles,
                                          tile_capacity, dx, O, I, s))
        return rc;
    // dw[e] (O, I) = dy[segment]^T . x[segment]: the dW2 product of the SwiGLU backward
    if (dw)
      return bf16_grouped_bwd(dy, nullptr, nullptr, 0, nullptr, nullptr, nullptr, nullptr, nullptr, x, nullptr, nullptr,
                              seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity, nullptr,
                              nullptr, nullptr, nullptr, nullptr, dw, El, O, I, 16, s);
    return MI355_OK;
  }
  // dx = dy . w[e]: B(k=o, n=i) = w[e][o][i]
  if (dx && rows)
    if (int rc = rowseg(sg, dy, O, w, I, 1, O * I, dx, I, O, dtype, 0, s)) return rc;
  // the weight gradient also covers the no-rows case: every expert's gradient is written (zeros)
  if (dw) return kseg(sg, dy, x, dw, O, I, El, dtype, s);
  return MI355_OK;
}

extern "C" int64_t mi355_grouped_combine_bwd_slots(int dtype, int64_t D, int64_t F) {
  if (dtype != MI355_BF16 || D < 1 || F < 1 || !bf16_fast_path_ok(D, F)) return 0;
  return bf16_fused_dot_slots(F);
}

extern "C" int mi355_grouped_swiglu_combine_bwd(
    const void* dout, const void* x, const int32_t* token_of_row, int64_t num_tokens, const float* row_scale,
    const void* w1, const void* w3, const void* w2, const void* gate, const void* up, int dtype,
    const int32_t* seg_offsets,
    const int32_t* seg_counts, const int32_t* tile_expert, const int32_t* tile_row0, const int32_t* num_tiles,
    int64_t tile_capacity, void* dgate, void* dup, void* hs, float* dot_partial, void* drows, void* dw1,
    void* dw3, void* dw2, int64_t El, int64_t D, int64_t F, int64_t row_capacity, int stages, void* stream) {
  if (int rc = check_common("grouped_swiglu_combine_bwd", dtype, El, D, F, row_capacity, tile_capacity)) return rc;
  if (mi355_grouped_combine_bwd_slots(dtype, D, F) == 0)
    return fail(MI355_EUNSUP, "grouped_swiglu_combine_bwd: needs bf16 with D and F multiples of 64 (>= 384); "
                              "use mi355_combine_bwd + mi355_grouped_swiglu_bwd instead");
  MI355_REQUIRE(seg_offsets && seg_counts && num_tiles, "grouped_swiglu_combine_bwd: null plan pointer");
  MI355_REQUIRE(stages >= 0 && (stages & ~0x7c) == 0, "grouped_swiglu_combine_bwd: stages must be 0 or a mask of the backward stages");
  if (row_capacity == 0 || tile_capacity == 0) {
    // no rows: the weight gradients are still defined (zeros); the plain entry point writes them
    return mi355_grouped_swiglu_bwd(dout, x, token_of_row, num_tokens, w1, w3, w2, gate, up, hs, dtype, seg_offsets, seg_counts,
                                    tile_expert, tile_row0, num_tiles, tile_capacity, dgate, dup, drows, dw1, dw3,
                                    dw2, El, D, F, row_capacity, stream);
  }
  MI355_REQUIRE(dout && x && token_of_row && row_scale && w1 && w3 && w2 && gate && up && dgate && dup && hs &&
                    dot_partial && tile_expert && tile_row0,
                "grouped_swiglu_combine_bwd: null pointer");
  if (int rc = check_gather("grouped_swiglu_combine_bwd", token_of_row, num_tokens, D, dtype)) return rc;
  return bf16_grouped_bwd(dout, x, token_of_row, num_tokens, w1, w3, w2, gate, up, hs, row_scale, dot_partial,
                          seg_offsets, seg_counts, tile_expert, tile_row0, num_tiles, tile_capacity, dgate, dup,
                          drows, dw1, dw3, dw2, El, D, F, stages ? stages : 0x7c, as_stream(stream));
}
