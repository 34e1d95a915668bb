// Token permutation: the expert-major plan and the row movers.
//
// Plan = a stable counting sort of the N = T*K assignment slots by expert id.
//   1. plan_rank    each wave walks 256 consecutive slots in 64-slot chunks; within
//                   a chunk a slot's rank among equal experts is counted with 64
//                   lane reads, and the running per-wave expert counts live in LDS
//                   (one writer per expert and chunk).  The four waves of a workgroup
//                   then add the counts of the waves before them: emits the rank of
//                   every slot inside its workgroup's 1024 slots and the workgroup's
//                   histogram.
//   2. plan_scan    one workgroup: per-expert exclusive scan of the workgroup
//                   histograms (ascending workgroup = ascending slot, which is what
//                   makes the sort stable), the padded segment offsets, and the MFMA
//                   tile list.
//   3. plan_rows    row = segment offset + workgroups-before + rank-in-workgroup,
//                   written both ways (row_of_slot, slot_of_row).
// The row movers are pure bandwidth kernels: one wave per token, 16-byte lanes.
#include "common.h"

namespace mi355 {
namespace {

constexpr int kSlotsPerWave = 256;
constexpr int kWavesPerBlock = 4;
constexpr int kSlotsPerBlock = kSlotsPerWave * kWavesPerBlock;
constexpr int kBatch = 16;  // histogram loads in flight per lane in the scan

__global__ __launch_bounds__(256) void plan_rank_kernel(const int64_t* __restrict__ ids, int N,
                                                        int E, int32_t* __restrict__ rank_in_block,
                                                        int32_t* __restrict__ block_hist,
                                                        int32_t* __restrict__ slot_of_row,
                                                        int32_t* __restrict__ token_of_row, int row_capacity) {
  extern __shared__ int32_t cnt[];  // [4][E]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  // rows that end up without a slot (padding, unused capacity) read -1: every row starts as -1 here
  // and the rows kernel overwrites the real ones (a launch of its own for this fill cost as much
  // as the rows kernel)
  for (int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x; i < row_capacity;
       i += static_cast<int64_t>(gridDim.x) * 256) {
    slot_of_row[i] = -1;
    if (token_of_row) token_of_row[i] = -1;
  }
  volatile int32_t* my = cnt + wave * E;
  for (int e = lane; e < E; e += kWave) my[e] = 0;
  __syncthreads();

  const int begin = (blockIdx.x * kWavesPerBlock + wave) * kSlotsPerWave;
  constexpr int kChunks = kSlotsPerWave / kWave;
  int e_of[kChunks], rank_of[kChunks];
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int slot = begin + c * kWave + lane;
    const bool valid = slot < N;
    int e = valid ? static_cast<int>(ids[slot]) : -1;
    if (e < 0 || e >= E) e = -1;  // an id outside [0, E) is not counted and gets no row
    // rank among the chunk's lower lanes with the same expert, and whether a higher lane
    // holds it too: 64 uniform-lane reads, no LDS round trip per distinct expert
    int below = 0, above = 0;
#pragma unroll 8
    for (int j = 0; j < kWave; ++j) {
      const int ej = __builtin_amdgcn_readlane(e, j);
      const int same = (ej == e) ? 1 : 0;
      below += (j < lane) ? same : 0;
      above += (j > lane) ? same : 0;
    }
    e_of[c] = e;
    rank_of[c] = 0;
    if (e >= 0) {
      const int base = my[e];
      rank_of[c] = base + below;
      __builtin_amdgcn_wave_barrier();
      if (above == 0) my[e] = base + below + 1;  // one writer per expert: its highest lane
    }
    __builtin_amdgcn_wave_barrier();
  }
  __syncthreads();
  // the slots of the waves before this one in the workgroup come first
#pragma unroll
  for (int c = 0; c < kChunks; ++c) {
    const int e = e_of[c];
    if (e < 0) continue;
    int before = 0;
    for (int w = 0; w < wave; ++w) before += cnt[w * E + e];
    rank_in_block[begin + c * kWave + lane] = rank_of[c] + before;
  }
  for (int e = threadIdx.x; e < E; e += 256) {
    int sum = 0;
#pragma unroll
    for (int w = 0; w < kWavesPerBlock; ++w) sum += cnt[w * E + e];
    block_hist[static_cast<int64_t>(blockIdx.x) * E + e] = sum;
  }
}

// One workgroup of 1024 lanes.  The per-expert scan over the workgroup histograms of
// plan_rank is split into `parts` contiguous ranges so its loads pipeline: pass 1 sums
// each range, a short serial scan joins them, pass 2 writes the exclusive prefixes.
__global__ __launch_bounds__(1024) void plan_scan_kernel(
    const int32_t* __restrict__ hist, int32_t* __restrict__ prefix, int num_hist, int E,
    int lo, int hi, int align, int tile_m, int32_t* __restrict__ counts_E,
    int32_t* __restrict__ seg_offsets, int32_t* __restrict__ seg_counts,
    int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
    int32_t* __restrict__ num_tiles, int tile_capacity, int parts) {
  extern __shared__ int32_t sh[];
  const int El = hi - lo;
  int32_t* part_sum = sh;                  // parts * E
  int32_t* cnt_sh = part_sum + parts * E;  // E
  int32_t* seg_off_sh = cnt_sh + E;        // El + 1
  int32_t* tile_off_sh = seg_off_sh + El + 1;  // El + 1
  int32_t* pad_sh = tile_off_sh + El + 1;      // El
  int32_t* nt_sh = pad_sh + El;                // El
  const int tid = threadIdx.x;
  const int per = (num_hist + parts - 1) / parts;

  for (int idx = tid; idx < E * parts; idx += blockDim.x) {
    const int e = idx % E, part = idx / E;
    const int w0 = part * per, w1 = min(num_hist, w0 + per);
    // sixteen loads in flight at a time: one at a time, each would wait out a full memory
    // round trip, and this workgroup has nothing else to hide it behind
    int sum = 0;
    for (int w = w0; w < w1; w += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = w + i < w1 ? hist[static_cast<int64_t>(w + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i) sum += v[i];
    }
    part_sum[part * E + e] = sum;
  }
  __syncthreads();
  for (int e = tid; e < E; e += blockDim.x) {
    int run = 0;
    for (int part = 0; part < parts; ++part) {
      const int c = part_sum[part * E + e];
      part_sum[part * E + e] = run;
      run += c;
    }
    cnt_sh[e] = run;
    counts_E[e] = run;
    if (e >= lo && e < hi) seg_counts[e - lo] = run;
  }
  __syncthreads();
  for (int idx = tid; idx < E * parts; idx += blockDim.x) {
    const int e = idx % E, part = idx / E;
    const int w0 = part * per, w1 = min(num_hist, w0 + per);
    int run = part_sum[part * E + e];
    for (int w = w0; w < w1; w += kBatch) {
      int v[kBatch];
#pragma unroll
      for (int i = 0; i < kBatch; ++i) v[i] = w + i < w1 ? hist[static_cast<int64_t>(w + i) * E + e] : 0;
#pragma unroll
      for (int i = 0; i < kBatch; ++i) {
        if (w + i < w1) prefix[static_cast<int64_t>(w + i) * E + e] = run;
        run += v[i];
      }
    }
  }
  // padded rows and tiles per local expert; then, for every expert (and one past the last), what
  // lies before it.  Each of these El + 1 sums runs over all El experts: the lanes of the
  // workgroup share them, several lanes per sum over a slice of the experts each, joined by
  // integer adds in LDS (with one lane per sum -- 129 busy lanes of 1024, 128 rounds of LDS
  // reads each -- this step was half of the kernel's time).
  int32_t* rank_sh = nt_sh + El;  // El + 1
  for (int j = tid; j < El; j += blockDim.x) {
    const int c = cnt_sh[lo + j];
    pad_sh[j] = c + ((align - (c % align)) % align);
    nt_sh[j] = (c + tile_m - 1) / tile_m;
  }
  for (int j = tid; j <= El; j += blockDim.x) seg_off_sh[j] = tile_off_sh[j] = rank_sh[j] = 0;
  __syncthreads();
  // ... and its place among the local experts by descending row count (ties to the lower
  // index): the order in which the weight-gradient kernels start their tiles, longest
  // contraction first
  const int sums = El + 1;
  const int lanes_per_sum = max(1, static_cast<int>(blockDim.x) / sums);
  const int slice = (El + lanes_per_sum - 1) / lanes_per_sum;
  for (int idx = tid; idx < sums * lanes_per_sum; idx += blockDim.x) {
    const int j = idx % sums, o0 = (idx / sums) * slice, o1 = min(El, o0 + slice);
    const int c = j < El ? cnt_sh[lo + j] : 0;
    int off = 0, toff = 0, rank = 0;
#pragma unroll 4
    for (int o = o0; o < o1; ++o) {
      const bool before = o < j;
      off += before ? pad_sh[o] : 0;
      toff += before ? nt_sh[o] : 0;
      const int co = cnt_sh[lo + o];
      rank += (co > c || (co == c && before)) ? 1 : 0;
    }
    atomicAdd(&seg_off_sh[j], off);
    atomicAdd(&tile_off_sh[j], toff);
    atomicAdd(&rank_sh[j], rank);
  }
  __syncthreads();
  for (int j = tid; j <= El; j += blockDim.x) {
    if (j < El) seg_counts[El + rank_sh[j]] = j;
    else *num_tiles = tile_off_sh[j] < tile_capacity ? tile_off_sh[j] : tile_capacity;
  }
  for (int j = tid; j <= El; j += blockDim.x) seg_offsets[j] = seg_off_sh[j];
  for (int j = tid; j < El; j += blockDim.x) {
    const int c = cnt_sh[lo + j];
    const int nt = (c + tile_m - 1) / tile_m;
    const int rows = even_tile_rows(c, tile_m);
    for (int i = 0; i < nt; ++i) {
      const int idx = tile_off_sh[j] + i;
      if (idx < tile_capacity) {
        tile_expert[idx] = j;
        tile_row0[idx] = seg_off_sh[j] + i * rows;
      }
    }
  }
}

// Segment offsets and tile list for rows that are already expert-major with the
// given per-expert row counts (the layout GroupedExperts.forward receives).
__global__ __launch_bounds__(256) void segments_from_counts_kernel(
    const int32_t* __restrict__ counts, int El, int tile_m, int row_capacity,
    int32_t* __restrict__ seg_offsets, int32_t* __restrict__ seg_counts,
    int32_t* __restrict__ tile_expert, int32_t* __restrict__ tile_row0,
    int32_t* __restrict__ num_tiles, int tile_capacity) {
  extern __shared__ int32_t sh[];
  int32_t* seg_off_sh = sh;
  int32_t* tile_off_sh = sh + El + 1;
  int32_t* cnt_sh = sh + 2 * El + 2;
  int32_t* raw_sh = cnt_sh + El;
  const int tid = threadIdx.x;
  // Clamped so that no segment reaches past the rows that exist: the offset of expert j is
  // min(sum of the counts before it, row_capacity) and it keeps what still fits -- what a
  // serial walk would give, computed by every lane for its own expert.
  for (int j = tid; j < El; j += blockDim.x) raw_sh[j] = max(counts[j], 0);
  __syncthreads();
  for (int j = tid; j <= El; j += blockDim.x) {
    int64_t before = 0;
#pragma unroll 16
    for (int o = 0; o < El; ++o) before += o < j ? raw_sh[o] : 0;
    const int off = static_cast<int>(min(before, static_cast<int64_t>(row_capacity)));
    seg_off_sh[j] = off;
    if (j < El) cnt_sh[j] = min(raw_sh[j], row_capacity - off);
  }
  __syncthreads();
  // tiles before each expert, and the experts by descending row count (ties to the lower
  // index): the order in which the weight-gradient kernels start their tiles
  for (int j = tid; j <= El; j += blockDim.x) {
    const int c = j < El ? cnt_sh[j] : 0;
    int toff = 0, rank = 0;
#pragma unroll 16
    for (int o = 0; o < El; ++o) {
      const int co = cnt_sh[o];
      const bool before = o < j;
      toff += before ? (co + tile_m - 1) / tile_m : 0;
      rank += (co > c || (co == c && before)) ? 1 : 0;
    }
    tile_off_sh[j] = toff;
    if (j < El) seg_counts[El + rank] = j;
    else *num_tiles = toff < tile_capacity ? toff : tile_capacity;
  }
  __syncthreads();
  for (int j = tid; j <= El; j += blockDim.x) seg_offsets[j] = seg_off_sh[j];
  for (int j = tid; j < El; j += blockDim.x) {
    const int c = cnt_sh[j];
    seg_counts[j] = c;
    const int nt = (c + tile_m - 1) / tile_m;
    const int rows = even_tile_rows(c, tile_m);
    for (int i = 0; i < nt; ++i) {
      const int idx = tile_off_sh[j] + i;
      if (idx < tile_capacity) {
        tile_expert[idx] = j;
        tile_row0[idx] = seg_off_sh[j] + i * rows;
      }
    }
  }
}

// p[0..n) = v, and q[0..n) too when q is given
__global__ void fill_i32_kernel(int32_t* p, int32_t* q, int64_t n, int32_t v) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < n) {
    p[i] = v;
    if (q) q[i] = v;
  }
}

__global__ __launch_bounds__(256) void plan_rows_kernel(
    const int64_t* __restrict__ ids, const int32_t* __restrict__ rank_in_block,
    const int32_t* __restrict__ block_prefix, const int32_t* __restrict__ seg_offsets, int N, int E,
    int lo, int hi, int K, int32_t* __restrict__ row_of_slot, int32_t* __restrict__ slot_of_row,
    int32_t* __restrict__ token_of_row, int row_capacity) {
  const int slot = blockIdx.x * blockDim.x + threadIdx.x;
  if (slot >= N) return;
  const int e = static_cast<int>(ids[slot]);  // outside [0, E): outside [lo, hi) too, no row
  int row = -1;
  if (e >= lo && e < hi) {
    const int blk = slot / kSlotsPerBlock;
    row = seg_offsets[e - lo] + block_prefix[static_cast<int64_t>(blk) * E + e] + rank_in_block[slot];
    if (row >= 0 && row < row_capacity) {
      slot_of_row[row] = slot;
      if (token_of_row) token_of_row[row] = slot / K;
    } else {
      row = -1;
    }
  }
  row_of_slot[slot] = row;
}

// ---- row movers ---------------------------------------------------------------
// 16-byte vectors when the row length allows, else scalars.
//
// rows[row_of_slot[t*K + k]] = x[t]: one wave per token reads the token row ONCE and stores its
// K copies (walking the rows instead re-fetches every token row K times from wherever it has
// gone meanwhile: 1.7x the algorithmic traffic at K = 8).  Waves past the tokens zero the
// padding rows (slot_of_row < 0) below *total_rows.
template <typename T>
__global__ __launch_bounds__(256) void permute_rows_fwd_kernel(
    const T* __restrict__ x, const int32_t* __restrict__ row_of_slot, const int32_t* __restrict__ slot_of_row,
    const int32_t* __restrict__ total_rows, T* __restrict__ rows, int T_, int D, int K, int token_blocks,
    int row_capacity, int stream_stores) {
  const int lane = threadIdx.x & 63;
  constexpr int V = 16 / sizeof(T);
  if (static_cast<int>(blockIdx.x) >= token_blocks) {
    const int r = (blockIdx.x - token_blocks) * 4 + (threadIdx.x >> 6);
    if (r >= row_capacity || r >= *total_rows || slot_of_row[r] >= 0) return;
    T* dst = rows + static_cast<int64_t>(r) * D;
    if (D % V == 0) {
      for (int i = lane; i < D / V; i += kWave) reinterpret_cast<uint4*>(dst)[i] = make_uint4(0, 0, 0, 0);
    } else {
      for (int i = lane; i < D; i += kWave) dst[i] = T(0);
    }
    return;
  }
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  const T* src = x + static_cast<int64_t>(t) * D;
  if (D % V == 0) {
    const int nv = D / V;
    constexpr int G = 4;  // vectors per lane and pass: 4 KiB of the row in flight per wave
    for (int base = 0; base < nv; base += G * kWave) {
      uint4 v[G];
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int i = base + g * kWave + lane;
        v[g] = i < nv ? reinterpret_cast<const uint4*>(src)[i] : make_uint4(0, 0, 0, 0);
      }
      for (int k = 0; k < K; ++k) {
        int row = row_of_slot[s0 + k];  // wave-uniform
        if (row < 0 || row >= row_capacity) continue;
        uint4* d4 = reinterpret_cast<uint4*>(rows + static_cast<int64_t>(row) * D);
#pragma unroll
        for (int g = 0; g < G; ++g) {
          const int i = base + g * kWave + lane;
          if (i < nv) {
            if (stream_stores) store_stream(d4 + i, v[g]);
            else d4[i] = v[g];
          }
        }
      }
    }
  } else {
    for (int i = lane; i < D; i += kWave) {
      const T v = src[i];
      for (int k = 0; k < K; ++k) {
        const int row = row_of_slot[s0 + k];
        if (row >= 0 && row < row_capacity) rows[static_cast<int64_t>(row) * D + i] = v;
      }
    }
  }
}

template <typename T>
__device__ __forceinline__ void acc_vec(float (&a)[16 / sizeof(T)], const uint4& v);
template <>
__device__ __forceinline__ void acc_vec<float>(float (&a)[4], const uint4& v) {
  a[0] += __uint_as_float(v.x); a[1] += __uint_as_float(v.y);
  a[2] += __uint_as_float(v.z); a[3] += __uint_as_float(v.w);
}
template <>
__device__ __forceinline__ void acc_vec<uint16_t>(float (&a)[8], const uint4& v) {
  a[0] += __uint_as_float(v.x << 16); a[1] += __uint_as_float(v.x & 0xffff0000u);
  a[2] += __uint_as_float(v.y << 16); a[3] += __uint_as_float(v.y & 0xffff0000u);
  a[4] += __uint_as_float(v.z << 16); a[5] += __uint_as_float(v.z & 0xffff0000u);
  a[6] += __uint_as_float(v.w << 16); a[7] += __uint_as_float(v.w & 0xffff0000u);
}
template <typename T>
__device__ __forceinline__ uint4 pack_vec(const float (&a)[16 / sizeof(T)]);
template <>
__device__ __forceinline__ uint4 pack_vec<float>(const float (&a)[4]) {
  return make_uint4(__float_as_uint(a[0]), __float_as_uint(a[1]), __float_as_uint(a[2]),
                    __float_as_uint(a[3]));
}
template <>
__device__ __forceinline__ uint4 pack_vec<uint16_t>(const float (&a)[8]) {
  return make_uint4(pack_bf16x2(a[0], a[1]), pack_bf16x2(a[2], a[3]), pack_bf16x2(a[4], a[5]),
                    pack_bf16x2(a[6], a[7]));
}

template <typename T>
__global__ __launch_bounds__(256) void permute_rows_bwd_kernel(
    const T* __restrict__ drows, const int32_t* __restrict__ row_of_slot, T* __restrict__ dx, int T_,
    int D, int K) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  constexpr int V = 16 / sizeof(T);
  T* dst = dx + static_cast<int64_t>(t) * D;
  const int my_row = lane < K ? row_of_slot[static_cast<int64_t>(t) * K + lane] : -1;  // K <= 64
  // Loops are uniform across the wave (shuffles need every lane); lanes past the
  // end of the row just skip their loads and stores.
  if (D % V == 0) {
    const int nv = D / V;
    // G vectors per lane and pass (4 KiB of every row per wave) from eight rows at a time, all
    // requested before the first is summed: 32 KiB in flight per wave.  The row numbers are
    // wave-uniform (scalar address arithmetic); the sum still runs in ascending k.
    constexpr int G = 4, B = 8;
    for (int base = 0; base < nv; base += G * kWave) {
      float a[G][V];
#pragma unroll
      for (int g = 0; g < G; ++g)
#pragma unroll
        for (int q = 0; q < V; ++q) a[g][q] = 0.0f;
      for (int k0 = 0; k0 < K; k0 += B) {
        uint4 v[B][G];
#pragma unroll
        for (int j = 0; j < B; ++j) {
          const int k = k0 + j;
          const int row = k < K ? __builtin_amdgcn_readfirstlane(__shfl(my_row, k, kWave)) : -1;
          const uint4* src = reinterpret_cast<const uint4*>(drows + static_cast<int64_t>(max(row, 0)) * D);
#pragma unroll
          for (int g = 0; g < G; ++g) {
            const int i = base + g * kWave + lane;
            v[j][g] = (row >= 0 && i < nv) ? load_stream(src + i) : make_uint4(0, 0, 0, 0);
          }
        }
#pragma unroll
        for (int j = 0; j < B; ++j)
#pragma unroll
          for (int g = 0; g < G; ++g) acc_vec<T>(a[g], v[j][g]);  // absent rows add zeros
      }
#pragma unroll
      for (int g = 0; g < G; ++g) {
        const int i = base + g * kWave + lane;
        if (i < nv) reinterpret_cast<uint4*>(dst)[i] = pack_vec<T>(a[g]);
      }
    }
  } else {
    for (int base = 0; base < D; base += kWave) {
      const int i = base + lane;
      const bool on = i < D;
      float a = 0.0f;
      for (int k = 0; k < K; ++k) {
        const int row = __shfl(my_row, k, kWave);
        if (row >= 0 && on) a += load_as_f32(drows + static_cast<int64_t>(row) * D + i);
      }
      if (on) store_from_f32(dst + i, a);
    }
  }
}

// fp64 rows: the K-way sum in fp64, ascending k, one wave per token
__global__ __launch_bounds__(256) void permute_rows_bwd_f64_kernel(
    const double* __restrict__ drows, const int32_t* __restrict__ row_of_slot, double* __restrict__ dx,
    int T_, int D, int K) {
  const int lane = threadIdx.x & 63;
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (t >= T_) return;
  const int64_t s0 = static_cast<int64_t>(t) * K;
  double* dst = dx + static_cast<int64_t>(t) * D;
  for (int i = lane; i < D; i += kWave) {
    double a = 0.0;
    for (int k = 0; k < K; ++k) {
      const int row = row_of_slot[s0 + k];  // wave-uniform
      if (row >= 0) a += drows[static_cast<int64_t>(row) * D + i];
    }
    dst[i] = a;
  }
}

}  // namespace
}  // namespace mi355

using namespace mi355;

static int64_t plan_num_blocks(int64_t N) { return (N + kSlotsPerBlock - 1) / kSlotsPerBlock; }

extern "C" int64_t mi355_permute_plan_workspace_bytes(int64_t T, int64_t K, int64_t E) {
  const int64_t N = T * K;
  // rank_in_block[N] + block_hist[blocks][E] + block_prefix[blocks][E]
  return (N + 2 * plan_num_blocks(N) * E + 64) * (int64_t)sizeof(int32_t);
}

static int plan_impl(const int64_t* ids, int64_t T, int64_t K, int64_t E, int64_t lo, int64_t hi, int64_t align,
                     int64_t tile_m, int32_t* counts_E, int32_t* seg_offsets, int32_t* seg_counts,
                     int32_t* row_of_slot, int32_t* slot_of_row, int32_t* token_of_row, int64_t row_capacity,
                     int32_t* tile_expert, int32_t* tile_row0, int32_t* num_tiles, int64_t tile_capacity,
                     void* workspace, hipStream_t s) {
  const int64_t N = T * K;
  MI355_REQUIRE(T >= 0 && K >= 1 && E >= 1 && N < (1ll << 30), "permute_plan: bad shape T=%lld K=%lld E=%lld",
                (long long)T, (long long)K, (long long)E);
  // (the scan workgroup keeps (parts + 1) * E + 5 * El + 3 words in LDS: 56 KiB at E = 2048)
  MI355_REQUIRE(E <= 2048, "permute_plan: E=%lld exceeds 2048", (long long)E);
  MI355_REQUIRE(0 <= lo && lo < hi && hi <= E, "permute_plan: bad local range [%lld,%lld)", (long long)lo, (long long)hi);
  MI355_REQUIRE(align >= 1 && tile_m >= 1, "permute_plan: align and tile_m must be positive");
  MI355_REQUIRE(row_capacity >= 0 && row_capacity < (1ll << 31) && tile_capacity >= 0,
                "permute_plan: bad capacity");
  MI355_REQUIRE(counts_E && seg_offsets && seg_counts && num_tiles && workspace,
                "permute_plan: null pointer");
  MI355_REQUIRE(N == 0 || (ids && row_of_slot), "permute_plan: null pointer");
  MI355_REQUIRE(row_capacity == 0 || slot_of_row, "permute_plan: null slot_of_row");
  int32_t* rank_in_block = static_cast<int32_t*>(workspace);
  int32_t* block_hist = rank_in_block + N;
  const int nblocks = (int)plan_num_blocks(N);
  if (nblocks > 0) {
    hipLaunchKernelGGL(plan_rank_kernel, dim3(nblocks), dim3(256), (size_t)kWavesPerBlock * E * 4, s,
                       ids, (int)N, (int)E, rank_in_block, block_hist, slot_of_row, token_of_row, (int)row_capacity);
    if (int rc = check_launch("plan_rank")) return rc;
  } else if (row_capacity > 0) {  // no slots at all: only the fill is left to do
    hipLaunchKernelGGL(fill_i32_kernel, dim3((unsigned)((row_capacity + 255) / 256)), dim3(256), 0, s,
                       slot_of_row, token_of_row, row_capacity, -1);
    if (int rc = check_launch("plan_fill")) return rc;
  }
  const int El = (int)(hi - lo);
  int32_t* block_prefix = block_hist + (int64_t)nblocks * E;
  int parts = (int)(1024 / E);
  if (parts < 1) parts = 1;
  if (parts > 16) parts = 16;
  hipLaunchKernelGGL(plan_scan_kernel, dim3(1), dim3(1024),
                     (size_t)((parts + 1) * E + 5 * El + 3) * 4, s, block_hist, block_prefix, nblocks,
                     (int)E, (int)lo, (int)hi, (int)align, (int)tile_m, counts_E, seg_offsets,
                     seg_counts, tile_expert, tile_row0, num_tiles, (int)tile_capacity, parts);
  if (int rc = check_launch("plan_scan")) return rc;
  if (N > 0) {
    hipLaunchKernelGGL(plan_rows_kernel, dim3((unsigned)((N + 255) / 256)), dim3(256), 0, s, ids,
                       rank_in_block, block_prefix, seg_offsets, (int)N, (int)E, (int)lo, (int)hi, (int)K,
                       row_of_slot, slot_of_row, token_of_row, (int)row_capacity);
    if (int rc = check_launch("plan_rows")) return rc;
  }
  return MI355_OK;
}

extern "C" int mi355_permute_plan(const int64_t* ids, int64_t T, int64_t K, int64_t E,
                                  int64_t lo, int64_t hi, int64_t align, int64_t tile_m,
                                  int32_t* counts_E, int32_t* seg_offsets, int32_t* seg_counts,
                                  int32_t* row_of_slot, int32_t* slot_of_row,
                                  int32_t* token_of_row, int64_t row_capacity, int32_t* tile_expert, int32_t* tile_row0,
                                  int32_t* num_tiles, int64_t tile_capacity, void* workspace,
                                  void* stream) {
  return plan_impl(ids, T, K, E, lo, hi, align, tile_m, counts_E, seg_offsets, seg_counts, row_of_slot, slot_of_row,
                   token_of_row, row_capacity, tile_expert, tile_row0, num_tiles, tile_capacity, workspace,
                   as_stream(stream));
}

// ---- the same plan without a caller-provided workspace -------------------------------------
// For callers that cannot allocate (under HIP graph capture, in a tight serving loop): the
// ranks and per-workgroup histograms live in a file-scope device array, 8 MiB per GPU, held until
// the process ends.  The array's name is a host-side stand-in, not a device address: its
// address on each device is asked for once, with that device current, and only that pointer
// is ever handed to kernels.  Every call on a GPU shares that GPU's array: calls that overlap
// on one GPU (two streams, two threads) race.  Nothing in it must start at zero -- every word
// a kernel of the plan reads was written by an earlier kernel of the same call.
constexpr int64_t kStaticPlanBytes = 8ll << 20;
static __device__ __align__(256) unsigned char plan_scratch[kStaticPlanBytes];
constexpr int kMaxDevices = 64;
static std::atomic<void*> plan_scratch_ptr[kMaxDevices];

extern "C" int64_t mi355_permute_plan_static_max_bytes(void) { return kStaticPlanBytes; }

extern "C" int mi355_permute_plan_static(const int64_t* ids, int64_t T, int64_t K, int64_t E, int64_t lo,
                                         int64_t hi, int64_t align, int64_t tile_m, int32_t* counts_E,
                                         int32_t* seg_offsets, int32_t* seg_counts, int32_t* row_of_slot,
                                         int32_t* slot_of_row, int32_t* token_of_row, int64_t row_capacity,
                                         int32_t* tile_expert, int32_t* tile_row0, int32_t* num_tiles,
                                         int64_t tile_capacity, void* stream) {
  MI355_REQUIRE(T >= 0 && K >= 1 && E >= 1 && T * K < (1ll << 30) && E <= 2048,
                "permute_plan_static: bad shape T=%lld K=%lld E=%lld", (long long)T, (long long)K, (long long)E);
  const int64_t need = mi355_permute_plan_workspace_bytes(T, K, E);
  MI355_REQUIRE(need <= kStaticPlanBytes,
                "permute_plan_static: T=%lld K=%lld E=%lld needs %lld bytes of scratch, the built-in array holds %lld; "
                "use mi355_permute_plan with a workspace of your own",
                (long long)T, (long long)K, (long long)E, (long long)need, (long long)kStaticPlanBytes);
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices)
    return fail(MI355_ELAUNCH, "permute_plan_static: no current device");
  void* ptr = plan_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    // The first call on a device resolves the array's address, which may load the code object:
    // not something to do while a stream records a graph.  A caller who captures calls this
    // entry point once, uncaptured, beforehand (any size; T = 0 will do).
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(as_stream(stream), &capturing) == hipSuccess && capturing != hipStreamCaptureStatusNone)
      return fail(MI355_EINVAL, "permute_plan_static: the first call on a device must not be under stream capture "
                                "(call it once before capturing)");
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(plan_scratch));
    if (e != hipSuccess || !ptr)
      return fail(MI355_ELAUNCH, "permute_plan_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
    plan_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  return plan_impl(ids, T, K, E, lo, hi, align, tile_m, counts_E, seg_offsets, seg_counts, row_of_slot, slot_of_row,
                   token_of_row, row_capacity, tile_expert, tile_row0, num_tiles, tile_capacity, ptr,
                   as_stream(stream));
}

extern "C" int mi355_permute_rows_fwd(const void* x, int dtype, const int32_t* row_of_slot,
                                      const int32_t* slot_of_row, const int32_t* total_rows, void* rows,
                                      int64_t T, int64_t D, int64_t K, int64_t row_capacity, void* stream) {
  MI355_REQUIRE(D >= 1 && K >= 1 && T >= 0 && T < (1ll << 31) && T * K < (1ll << 31) && row_capacity >= 0 &&
                    row_capacity < (1ll << 31) && D < (1ll << 31),
                "permute_rows_fwd: bad shape");
  if (row_capacity == 0) return MI355_OK;
  if (dtype == MI355_F64) {
    // a copy moves bytes: an fp64 row is an fp32 row of twice the length
    MI355_REQUIRE(D < (1ll << 30), "permute_rows_fwd: bad shape");
    dtype = MI355_F32;
    D *= 2;
  }
  MI355_REQUIRE(rows && (T == 0 || (x && row_of_slot)), "permute_rows_fwd: null pointer");
  MI355_REQUIRE(!slot_of_row || total_rows, "permute_rows_fwd: total_rows required with slot_of_row");
  const int token_blocks = (int)((T + 3) / 4);
  const int pad_blocks = slot_of_row ? (int)((row_capacity + 3) / 4) : 0;
  if (token_blocks + pad_blocks == 0) return MI355_OK;
  const dim3 grid((unsigned)(token_blocks + pad_blocks));
  // Rows that the 256 MiB memory-side cache can hold are written with plain stores and wait
  // there for the kernel that reads them (6.5 against 5.5 TB/s with non-temporal stores at
  // exactly 256 MiB); beyond that size they only displace each other, and non-temporal stores
  // are the faster ones (5.5 against 5.0 TB/s at 512 MiB).
  const int stream_stores = row_capacity * D * (dtype == MI355_F32 ? 4 : 2) > (256ll << 20);
  if (dtype == MI355_F32)
    hipLaunchKernelGGL(permute_rows_fwd_kernel<float>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const float*>(x), row_of_slot, slot_of_row, total_rows,
                       static_cast<float*>(rows), (int)T, (int)D, (int)K, token_blocks, (int)row_capacity, stream_stores);
  else if (dtype == MI355_BF16)
    hipLaunchKernelGGL(permute_rows_fwd_kernel<uint16_t>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t*>(x), row_of_slot, slot_of_row, total_rows,
                       static_cast<uint16_t*>(rows), (int)T, (int)D, (int)K, token_blocks, (int)row_capacity, stream_stores);
  else
    return fail(MI355_EINVAL, "permute_rows_fwd: unknown dtype %d", dtype);
  return check_launch("permute_rows_fwd");
}

extern "C" int mi355_permute_rows_bwd(const void* drows, int dtype, const int32_t* row_of_slot,
                                      void* dx, int64_t T, int64_t D, int64_t K, void* stream) {
  MI355_REQUIRE(D >= 1 && K >= 1 && K <= 64 && T >= 0 && T < (1ll << 31) && D < (1ll << 31),
                "permute_rows_bwd: bad shape (K must be <= 64)");
  if (T == 0) return MI355_OK;
  MI355_REQUIRE(row_of_slot && dx, "permute_rows_bwd: null pointer");
  const dim3 grid((unsigned)((T + 3) / 4));
  if (dtype == MI355_F32)
    hipLaunchKernelGGL(permute_rows_bwd_kernel<float>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const float*>(drows), row_of_slot, static_cast<float*>(dx),
                       (int)T, (int)D, (int)K);
  else if (dtype == MI355_BF16)
    hipLaunchKernelGGL(permute_rows_bwd_kernel<uint16_t>, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const uint16_t*>(drows), row_of_slot,
                       static_cast<uint16_t*>(dx), (int)T, (int)D, (int)K);
  else if (dtype == MI355_F64)
    hipLaunchKernelGGL(permute_rows_bwd_f64_kernel, grid, dim3(256), 0, as_stream(stream),
                       static_cast<const double*>(drows), row_of_slot, static_cast<double*>(dx), (int)T, (int)D,
                       (int)K);
  else
    return fail(MI355_EINVAL, "permute_rows_bwd: unknown dtype %d", dtype);
  return check_launch("permute_rows_bwd");
}

extern "C" int mi355_segments_from_counts(const int32_t* counts, int64_t El, int64_t tile_m,
                                          int64_t row_capacity, int32_t* seg_offsets, int32_t* seg_counts,
                                          int32_t* tile_expert, int32_t* tile_row0,
                                          int32_t* num_tiles, int64_t tile_capacity, void* stream) {
  MI355_REQUIRE(El >= 1 && El <= 8192 && tile_m >= 1 && tile_capacity >= 0 && row_capacity >= 0 &&
                    row_capacity < (1ll << 31),
                "segments_from_counts: bad shape El=%lld", (long long)El);
  MI355_REQUIRE(counts && seg_offsets && seg_counts && num_tiles, "segments_from_counts: null pointer");
  MI355_REQUIRE(tile_capacity == 0 || (tile_expert && tile_row0), "segments_from_counts: null tile list");
  hipLaunchKernelGGL(segments_from_counts_kernel, dim3(1), dim3(256), (size_t)(4 * El + 2) * 4,
                     as_stream(stream), counts, (int)El, (int)tile_m, (int)row_capacity, seg_offsets, seg_counts,
                     tile_expert, tile_row0, num_tiles, (int)tile_capacity);
  return check_launch("segments_from_counts");
}
