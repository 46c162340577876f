// The scale -> mask -> softmax chain of an attention block in one pass over
// the scores (the reference runs InPlaceProdScalar, InPlaceMask and Softmax as
// three nodes: ginn/node/inplace.h:104-123 and :152-212, ginn/nonlin.h:162-188),
// forward and backward.  Every intermediate is rounded to the storage type
// where the three separate kernels would have stored it, so the results are
// the same (for half storage: up to the last bit of a few results per million,
// where the compiler converts a product with one rounding in one kernel and
// with two in the other); the scores are read once, each result written once.
#include "common.h"
#include "kernel_util.h"
#include "vec_access.h"
#include "softmax_cols.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

template <typename T>
__device__ __forceinline__ float stored(float v) {
  return to_float<T>(from_float<T>(v));
}

// x[:, c] <- scale * x[:, c]; x[r, c] <- fill where mask[(c * rows + r) % mask_n] == 0;
// y[:, c] = softmax(x[:, c]).  One wave per column, the column in registers;
// rows % 8 == 0 and mask_n % rows == 0 (a column never straddles the mask's end).
template <typename T, int I, int U>
__global__ __launch_bounds__(kBlock) void scaled_masked_softmax_fwd_kernel(
    int rows, int cols, typename T::storage* x, float scale, const typename T::storage* __restrict__ mask,
    size_t mask_n, float fill, typename T::storage* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c0 = wave * U; c0 < cols; c0 += nwaves * U) {
    softmax_cols::Column<T, I> col[U];
    float m[U][I][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u < cols ? c0 + u : cols - 1;  // past the end: computed, not stored
      const size_t base = static_cast<size_t>(c) * rows;
      col[u].load(x + base, rows, lane);
      const size_t mbase = base % mask_n;
#pragma unroll
      for (int j = 0; j < I; ++j) {
        const int r = (j * 64 + lane) * 8;
        if (r < rows) {
          ld<T, 8>(mask + mbase + r, m[u][j]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) m[u][j][e] = 1.f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int j = 0; j < I; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          float v = stored<T>(scale * col[u].v[j][e]);
          if ((j * 64 + lane) * 8 >= rows) v = -INFINITY;  // past the end: neither maximum nor sum, whatever the scale
          col[u].v[j][e] = m[u][j][e] == 0.f ? stored<T>(fill) : v;
        }
      if (c0 + u < cols) col[u].store(x + static_cast<size_t>(c0 + u) * rows, rows, lane);
      float mx, inv;
      col[u].softmax(mx, inv);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (c0 + u < cols) col[u].store(y + static_cast<size_t>(c0 + u) * rows, rows, lane);
  }
}

// dx[:, c] = scale * (mask ? y (*) (dy - sum_rows(y (*) dy)) : 0), with the
// roundings of softmax backward, mask and scale as separate kernels.
template <typename T, int I, int U>
__global__ __launch_bounds__(kBlock) void scaled_masked_softmax_bwd_kernel(
    int rows, int cols, const typename T::storage* __restrict__ dy, const typename T::storage* __restrict__ y,
    float scale, const typename T::storage* __restrict__ mask, size_t mask_n, typename T::storage* __restrict__ dx) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c0 = wave * U; c0 < cols; c0 += nwaves * U) {
    float yv[U][I][8], gv[U][I][8], m[U][I][8];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u < cols ? c0 + u : cols - 1;
      const size_t base = static_cast<size_t>(c) * rows;
      const size_t mbase = base % mask_n;
#pragma unroll
      for (int j = 0; j < I; ++j) {
        const int r = (j * 64 + lane) * 8;
        if (r < rows) {
          ld<T, 8>(y + base + r, yv[u][j]);
          ld<T, 8>(dy + base + r, gv[u][j]);
          ld<T, 8>(mask + mbase + r, m[u][j]);
        } else {
#pragma unroll
          for (int e = 0; e < 8; ++e) yv[u][j][e] = gv[u][j][e] = m[u][j][e] = 0.f;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float dot = 0.f;
#pragma unroll
      for (int j = 0; j < I; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) dot += yv[u][j][e] * gv[u][j][e];
      dot = wave_sum(dot);
#pragma unroll
      for (int j = 0; j < I; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const float g = stored<T>(yv[u][j][e] * (gv[u][j][e] - dot));
          gv[u][j][e] = scale * (m[u][j][e] == 0.f ? 0.f : g);
        }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (c0 + u >= cols) continue;
      const size_t base = static_cast<size_t>(c0 + u) * rows;
#pragma unroll
      for (int j = 0; j < I; ++j) {
        const int r = (j * 64 + lane) * 8;
        if (r < rows) st<T, 8>(dx + base + r, gv[u][j]);
      }
    }
  }
}

// Runs CALL with I bound to `vectors` (1, 2 or 4).
#define GH_DISPATCH_SHORT_COLUMN(vectors, CALL)     \
  switch (vectors) {                                \
    case 1: { constexpr int I = 1; CALL; } break;   \
    case 2: { constexpr int I = 2; CALL; } break;   \
    default: { constexpr int I = 4; CALL; } break;  \
  }

// Shapes the one-pass kernels take: whole 16-byte vectors per column, the
// column in at most 4 vectors per lane (register budget with the mask and, in
// backward, two operands held as well), the mask covering whole columns.
bool one_pass(int rows, size_t mask_n, std::initializer_list<const void*> ptrs) {
  if (rows % 8 != 0 || rows > 64 * 8 * 4 || mask_n % static_cast<size_t>(rows) != 0) return false;
  return vec8_ok(ptrs, {static_cast<size_t>(rows)});
}

}  // namespace
}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_scaled_masked_softmax_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, void* x,
                                       float scale, const void* mask, size_t mask_n, float fill, void* y) {
  GH_CHECK_ARG(ctx, "ginn_hip_scaled_masked_softmax_fwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_scaled_masked_softmax_fwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && mask && y, "ginn_hip_scaled_masked_softmax_fwd: NULL pointer");
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_CHECK_ARG(mask_n > 0 && n % mask_n == 0,
               "ginn_hip_scaled_masked_softmax_fwd: the mask's size (%zu) does not divide the operand's (%zu)", mask_n, n);
  GH_CHECK_ARG(x != y, "ginn_hip_scaled_masked_softmax_fwd: x and y must be different arrays");
  GH_HIP(hipSetDevice(ctx->device));
  if (one_pass(rows, mask_n, {x, mask, y})) {
    GH_DISPATCH_SHORT_COLUMN(softmax_cols::vectors_for(rows), {
      constexpr int U = I == 1 ? 2 : 1;
      const unsigned grid = grid_for((cols + U - 1) / U, kBlock / 64, ctx->num_cus);
      GH_DISPATCH_DTYPE(dtype, (scaled_masked_softmax_fwd_kernel<T, I, U><<<grid, kBlock, 0, ctx->stream>>>(
          rows, cols, static_cast<T::storage*>(x), scale, static_cast<const T::storage*>(mask), mask_n, fill,
          static_cast<T::storage*>(y))));
    });
    GH_HIP(hipGetLastError());
    return kOk;
  }
  // Any other shape: the three steps one after the other.
  int rc = ginn_hip_scale_shift(ctx, dtype, n, scale, 0.f, x, x, 0);
  if (rc == kOk) rc = ginn_hip_mask_fill(ctx, dtype, mask_n, n / mask_n, mask, fill, x);
  if (rc == kOk) rc = ginn_hip_nonlin_fwd(ctx, dtype, GINN_HIP_ACT_SOFTMAX, rows, cols, x, y);
  return rc;
}

int ginn_hip_scaled_masked_softmax_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* dy,
                                       const void* y, float scale, const void* mask, size_t mask_n, void* dx) {
  GH_CHECK_ARG(ctx, "ginn_hip_scaled_masked_softmax_bwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_scaled_masked_softmax_bwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(dy && y && mask && dx, "ginn_hip_scaled_masked_softmax_bwd: NULL pointer");
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_CHECK_ARG(mask_n > 0 && n % mask_n == 0,
               "ginn_hip_scaled_masked_softmax_bwd: the mask's size (%zu) does not divide the operand's (%zu)", mask_n, n);
  GH_CHECK_ARG(dx != dy && dx != y, "ginn_hip_scaled_masked_softmax_bwd: dx must not be an input");
  GH_HIP(hipSetDevice(ctx->device));
  if (one_pass(rows, mask_n, {dy, y, mask, dx})) {
    GH_DISPATCH_SHORT_COLUMN(softmax_cols::vectors_for(rows), {
      constexpr int U = I == 1 ? 2 : 1;
      const unsigned grid = grid_for((cols + U - 1) / U, kBlock / 64, ctx->num_cus);
      GH_DISPATCH_DTYPE(dtype, (scaled_masked_softmax_bwd_kernel<T, I, U><<<grid, kBlock, 0, ctx->stream>>>(
          rows, cols, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(y), scale,
          static_cast<const T::storage*>(mask), mask_n, static_cast<T::storage*>(dx))));
    });
    GH_HIP(hipGetLastError());
    return kOk;
  }
  int rc = ginn_hip_nonlin_bwd(ctx, dtype, GINN_HIP_ACT_SOFTMAX, rows, cols, dy, nullptr, y, dx, 0);
  if (rc == kOk) rc = ginn_hip_mask_fill(ctx, dtype, mask_n, n / mask_n, mask, 0.f, dx);
  if (rc == kOk) rc = ginn_hip_scale_shift(ctx, dtype, n, scale, 0.f, dx, dx, 0);
  return rc;
}

}  // extern "C"
