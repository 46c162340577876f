// Shared geometry for kernels that walk the columns of a column-major
// [rows x cols] matrix and leave per-row sums: a block owns 64 V consecutive
// rows (V per lane: 8 = 16-byte accesses when rows and pointers allow, else 1;
// a wave reads consecutive addresses either way) and a chunk of columns; its 4
// waves take every 4th column of the chunk and combine through LDS.  Per-chunk
// fp32 partials are folded by fold_rows_kernel, which spreads the chunks of a
// row over 64 threads.
#ifndef GINN_HIP_REDUCE_ROWS_H
#define GINN_HIP_REDUCE_ROWS_H

#include "common.h"

namespace ginn_hip {
namespace rowred {

constexpr int kBlock = 256;
constexpr int kRowsPerBlock = 64;
constexpr int kSlices = kBlock / kRowsPerBlock;  // waves per block = column phases
constexpr int kMaxChunks = 128;
// The fold: a block of 1024 threads owns 16 rows and spreads their chunks over
// 64 slices (the fold is pure latency: few bytes, many loads in flight).
constexpr int kFoldBlock = 1024;
constexpr int kFoldRows = 16;
constexpr int kFoldSlices = kFoldBlock / kFoldRows;

struct Plan {
  int row_blocks;   // grid.x of the partial kernel (64 V rows each)
  int fold_blocks;  // grid.x of fold_rows_kernel (64 rows each)
  int chunks, cols_per_chunk;
};

// `sums` fp32 partial arrays of [chunks][rows] must fit the workspace;
// returns chunks = 0 when not even one chunk does.
inline Plan plan(int rows, int cols, int num_cus, size_t workspace_bytes, int sums, int rows_per_lane = 1) {
  Plan p;
  const int per_block = kRowsPerBlock * rows_per_lane;
  p.row_blocks = (rows + per_block - 1) / per_block;
  p.fold_blocks = (rows + kFoldRows - 1) / kFoldRows;
  int chunks = (num_cus * 4 + p.row_blocks - 1) / p.row_blocks;
  if (chunks > kMaxChunks) chunks = kMaxChunks;
  if (chunks > (cols + 4 * kSlices - 1) / (4 * kSlices)) chunks = (cols + 4 * kSlices - 1) / (4 * kSlices);
  if (chunks < 1) chunks = 1;
  const size_t per = static_cast<size_t>(sums) * rows * sizeof(float);
  if (per * chunks > workspace_bytes) chunks = static_cast<int>(workspace_bytes / per);
  if (chunks < 1) {
    p.chunks = 0;
    p.cols_per_chunk = 0;
    return p;
  }
  p.cols_per_chunk = cols > 0 ? (cols + chunks - 1) / chunks : 1;
  p.chunks = cols > 0 ? (cols + p.cols_per_chunk - 1) / p.cols_per_chunk : 1;
  return p;
}

// Combines the 4 waves' values of one row; valid in wave 0 afterwards.
__device__ __forceinline__ float combine(float v, float (*red)[kRowsPerBlock]) {
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  red[ty][tx] = v;
  __syncthreads();
  float s = 0.f;
  if (ty == 0) {
#pragma unroll
    for (int k = 0; k < kSlices; ++k) s += red[k][tx];
  }
  __syncthreads();
  return s;
}

// The same for V values per lane (rows tx V .. tx V + V - 1); red holds
// kSlices x V x 64 floats, value e of lane tx at [slice][e][tx].
template <int V>
__device__ __forceinline__ void combine_v(float (&v)[V], float* red) {
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
#pragma unroll
  for (int e = 0; e < V; ++e) red[(ty * V + e) * 64 + tx] = v[e];
  __syncthreads();
  if (ty == 0) {
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float s = 0.f;
#pragma unroll
      for (int k = 0; k < kSlices; ++k) s += red[(k * V + e) * 64 + tx];
      v[e] = s;
    }
  }
  __syncthreads();
}

// dst[r] (+)= sum over chunks of partial[c][r], for up to two partial arrays:
// slice s of a block's 64 takes the chunks s, s + 64, ...; the slices combine
// through LDS in index order.
template <typename T>
__device__ __forceinline__ void fold_rows_block(int block, int rows, int chunks, const float* __restrict__ part_a,
                                                const float* __restrict__ part_b, typename T::storage* dst_a,
                                                typename T::storage* dst_b, int accumulate,
                                                float (*red)[kFoldSlices][kFoldRows]) {
  const int tx = threadIdx.x % kFoldRows, ty = threadIdx.x / kFoldRows;
  const int r = block * kFoldRows + tx;
  float sa = 0.f, sb = 0.f;
  if (r < rows) {
#pragma unroll 4
    for (int c = ty; c < chunks; c += kFoldSlices) {
      if (dst_a) sa += part_a[static_cast<size_t>(c) * rows + r];
      if (dst_b) sb += part_b[static_cast<size_t>(c) * rows + r];
    }
  }
  red[0][ty][tx] = sa;
  red[1][ty][tx] = sb;
  __syncthreads();
  if (ty == 0 && r < rows) {
    sa = sb = 0.f;
#pragma unroll
    for (int k = 0; k < kFoldSlices; ++k) {
      sa += red[0][k][tx];
      sb += red[1][k][tx];
    }
    if (dst_a) dst_a[r] = from_float<T>((accumulate ? to_float<T>(dst_a[r]) : 0.f) + sa);
    if (dst_b) dst_b[r] = from_float<T>((accumulate ? to_float<T>(dst_b[r]) : 0.f) + sb);
  }
}

template <typename T>
__global__ __launch_bounds__(kFoldBlock) void fold_rows_kernel(int rows, int chunks, const float* __restrict__ part_a,
                                                               const float* __restrict__ part_b,
                                                               typename T::storage* dst_a, typename T::storage* dst_b,
                                                               int accumulate) {
  __shared__ float red[2][kFoldSlices][kFoldRows];
  fold_rows_block<T>(blockIdx.x, rows, chunks, part_a, part_b, dst_a, dst_b, accumulate, red);
}

// ---- who folds, and when ----------------------------------------------------
// A row-reduction entry point asks for room for its partial sums and hands the
// fold over:
//   Partials p = take_partials(ctx, bytes);      (ctx->mutex held)
//   ... launch the kernel that writes p.base ...
//   finish(ctx, job, p.deferred);
// Normally the room is the context's workspace and finish() launches
// fold_rows_kernel.  While the calling thread has asked for it
// (ginn_hip_defer_folds) the partial sums go to an area of their own, the job
// is queued, and flush_folds() folds everything queued in one launch.
struct Partials {
  float* base;
  bool deferred;
};
Partials take_partials(ginn_hip_ctx* ctx, size_t bytes);
int finish(ginn_hip_ctx* ctx, const ginn_hip_fold_job& job, bool deferred);
int flush_folds(ginn_hip_ctx* ctx);  // ctx->mutex held

}  // namespace rowred
}  // namespace ginn_hip

#endif  // GINN_HIP_REDUCE_ROWS_H
