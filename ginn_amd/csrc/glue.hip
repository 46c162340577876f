// Data-movement and elementwise companions of the product path: fills, strided
// copies, N-ary adds, broadcasts, reductions and the softmax + NLL loss head.
// All are bandwidth-bound, one pass over their operands.
#include "common.h"
#include "reduce_rows.h"
#include "kernel_util.h"
#include "vec_access.h"
#include "softmax_cols.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

// Grid-stride loop over n elements in steps of V per thread.
#define GH_GRID_STRIDE_V(i, n, V)                                              \
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * (V), \
              stride__ = static_cast<size_t>(gridDim.x) * kBlock * (V);        \
       i < (n); i += stride__)
#define GH_GRID_STRIDE(i, n) GH_GRID_STRIDE_V(i, n, 1)

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void fill_kernel(typename T::storage* dst, size_t n, float value) {
  float v[V];
#pragma unroll
  for (int e = 0; e < V; ++e) v[e] = value;
  GH_GRID_STRIDE_V(i, n, V) st<T, V>(dst + i, v);
}

// rows, lds and ldd are multiples of V when V > 1.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void copy_2d_kernel(int rows, int cols,
                                                         const typename T::storage* __restrict__ src, int lds,
                                                         typename T::storage* dst, int ldd, int accumulate) {
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_GRID_STRIDE_V(i, n, V) {
    const int r = static_cast<int>(i % rows);
    const size_t c = i / rows;
    float v[V];
    ld<T, V>(src + c * lds + r, v);
    if (accumulate) {
      float old[V];
      ld<T, V>(dst + c * ldd + r, old);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] += old[e];
    }
    st<T, V>(dst + c * ldd + r, v);
  }
}

struct AddSrcs {
  const void* p[8];
};

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void add_n_kernel(size_t n, int count, AddSrcs srcs,
                                                       typename T::storage* dst, int accumulate) {
  using S = typename T::storage;
  GH_GRID_STRIDE_V(i, n, V) {
    float v[V];
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = 0.f;
    if (accumulate) ld<T, V>(dst + i, v);
    for (int k = 0; k < count; ++k) {
      float t[V];
      ld<T, V>(static_cast<const S*>(srcs.p[k]) + i, t);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] += t[e];
    }
    st<T, V>(dst + i, v);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void cwise_prod_kernel(size_t n, const typename T::storage* __restrict__ a,
                                                            const typename T::storage* __restrict__ b,
                                                            typename T::storage* dst, int accumulate) {
  GH_GRID_STRIDE_V(i, n, V) {
    float x[V], y[V], old[V];
    ld<T, V>(a + i, x);
    ld<T, V>(b + i, y);
#pragma unroll
    for (int e = 0; e < V; ++e) old[e] = 0.f;
    if (accumulate) ld<T, V>(dst + i, old);
#pragma unroll
    for (int e = 0; e < V; ++e) x[e] = x[e] * y[e] + old[e];
    st<T, V>(dst + i, x);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void scale_shift_kernel(size_t n, float alpha, float shift,
                                                             const typename T::storage* x,
                                                             typename T::storage* dst, int accumulate) {
  GH_GRID_STRIDE_V(i, n, V) {
    float v[V], old[V];
    ld<T, V>(x + i, v);
#pragma unroll
    for (int e = 0; e < V; ++e) old[e] = 0.f;
    if (accumulate) ld<T, V>(dst + i, old);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] = alpha * v[e] + shift + old[e];
    st<T, V>(dst + i, v);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void col_broadcast_kernel(int rows, int cols,
                                                               const typename T::storage* __restrict__ x,
                                                               typename T::storage* dst) {
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_GRID_STRIDE_V(i, n, V) {
    float v[V];
    ld<T, V>(x + i % rows, v);
    st<T, V>(dst + i, v);
  }
}

// Row sums over the columns: per-chunk fp32 partials, folded by a second launch.
template <typename T, int V>
__global__ __launch_bounds__(rowred::kBlock) void row_sum_partial_kernel(int nrows, int cols, int cols_per_chunk,
                                                                       const typename T::storage* __restrict__ x,
                                                                       float* __restrict__ partial) {
  __shared__ float red[rowred::kSlices * V * 64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int r = (blockIdx.x * rowred::kRowsPerBlock + tx) * V;
  const int c0 = blockIdx.y * cols_per_chunk;
  const int c1 = min(cols, c0 + cols_per_chunk);
  float s[V];
#pragma unroll
  for (int e = 0; e < V; ++e) s[e] = 0.f;
  if (r < nrows)
#pragma unroll 4
    for (int c = c0 + ty; c < c1; c += rowred::kSlices) {
      float v[V];
      ld<T, V>(x + static_cast<size_t>(c) * nrows + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) s[e] += v[e];
    }
  rowred::combine_v<V>(s, red);
  if (ty == 0 && r < nrows) {
#pragma unroll
    for (int e = 0; e < V; ++e) partial[static_cast<size_t>(blockIdx.y) * nrows + r + e] = s[e];
  }
}

constexpr size_t kSumSmall = 16384;  // elements one block sums by itself

template <typename T>
__global__ __launch_bounds__(kBlock) void sum_partial_kernel(size_t n, const typename T::storage* __restrict__ x,
                                                             float* __restrict__ partial) {
  __shared__ float ws[kBlock / 64];
  float s = 0.f;
  GH_GRID_STRIDE(i, n) s += to_float<T>(x[i]);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) t += ws[w];
    partial[blockIdx.x] = t;
  }
}
// A short vector: one block does the whole sum and writes the result.
template <typename T>
__global__ __launch_bounds__(kBlock) void sum_small_kernel(size_t n, const typename T::storage* __restrict__ x,
                                                           float scale, typename T::storage* dst) {
  __shared__ float ws[kBlock / 64];
  // Four loads in flight per thread: the sum is a chain of memory latencies.
  float s4[4] = {0.f, 0.f, 0.f, 0.f};
  size_t i = threadIdx.x;
  for (; i + 3 * kBlock < n; i += 4 * kBlock) {
    float v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = to_float<T>(x[i + u * kBlock]);
#pragma unroll
    for (int u = 0; u < 4; ++u) s4[u] += v[u];
  }
  for (; i < n; i += kBlock) s4[0] += to_float<T>(x[i]);
  float s = wave_sum((s4[0] + s4[1]) + (s4[2] + s4[3]));
  if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) t += ws[w];
    dst[0] = from_float<T>(t * scale);
  }
}
template <typename T>
__global__ __launch_bounds__(64) void sum_fold_kernel(int blocks, const float* __restrict__ partial, float scale,
                                                      typename T::storage* dst) {
  float s = 0.f;
  for (int i = threadIdx.x; i < blocks; i += 64) s += partial[i];
  s = wave_sum(s);
  if (threadIdx.x == 0) dst[0] = from_float<T>(s * scale);
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void add_scalar_bcast_kernel(size_t n, const typename T::storage* __restrict__ src,
                                                                  float scale, typename T::storage* dst) {
  const float s = scale * to_float<T>(src[0]);
  GH_GRID_STRIDE_V(i, n, V) {
    float v[V];
    ld<T, V>(dst + i, v);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] += s;
    st<T, V>(dst + i, v);
  }
}

// Softmax + negative log-likelihood, one wave per column.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void pick_nls_fwd_kernel(int rows, int cols,
                                                              const typename T::storage* __restrict__ x,
                                                              const int* __restrict__ idx,
                                                              typename T::storage* __restrict__ smax,
                                                              float* __restrict__ stats,
                                                              typename T::storage* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float mx = -INFINITY;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) mx = fmaxf(mx, v[e]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) sum += softmax_exp<T>(v[e] - mx);
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int r = lane * V; smax && r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = softmax_exp<T>(v[e] - mx) * inv;
      st<T, V>(smax + base + r, v);
    }
    if (stats && lane == 0) {
      stats[2 * c] = mx;
      stats[2 * c + 1] = inv;
    }
    if (lane == 0) {
      // -log of the value as stored, as the reference picks from the stored
      // softmax (ginn/node/pick.h:182-186,213-214).
      const float picked = to_float<T>(from_float<T>(softmax_exp<T>(to_float<T>(x[base + idx[c]]) - mx) * inv));
      out[c] = from_float<T>(-logf(picked));
    }
  }
}

// The same with the column in registers (softmax_cols.h): the logits are read once.
template <typename T, int I>
__global__ __launch_bounds__(kBlock) void pick_nls_fwd_regs_kernel(int rows, int cols,
                                                                   const typename T::storage* __restrict__ x,
                                                                   const int* __restrict__ idx,
                                                                   typename T::storage* __restrict__ smax,
                                                                   float* __restrict__ stats,
                                                                   typename T::storage* __restrict__ out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    softmax_cols::Column<T, I> col;
    col.load(x + base, rows, lane);
    float picked_x = 0.f;
    if (lane == 0) picked_x = to_float<T>(x[base + idx[c]]);
    float mx, inv;
    col.softmax(mx, inv);
    if (smax) col.store(smax + base, rows, lane);
    if (stats && lane == 0) {
      stats[2 * c] = mx;
      stats[2 * c + 1] = inv;
    }
    if (lane == 0) {
      const float picked = to_float<T>(from_float<T>(softmax_exp<T>(picked_x - mx) * inv));
      out[c] = from_float<T>(-logf(picked));
    }
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void pick_nls_bwd_kernel(int rows, int cols,
                                                              const typename T::storage* __restrict__ smax,
                                                              const int* __restrict__ idx,
                                                              const typename T::storage* __restrict__ dout,
                                                              typename T::storage* dx, int accumulate) {
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_GRID_STRIDE_V(i, n, V) {
    const int r = static_cast<int>(i % rows);
    const int c = static_cast<int>(i / rows);
    const float g = to_float<T>(dout[c]);
    const int hot = idx[c] - r;  // position of the picked row inside this vector, if any
    float v[V], sm[V];
    if (accumulate) {
      ld<T, V>(dx + i, v);
    } else {
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = 0.f;
    }
    ld<T, V>(smax + i, sm);
#pragma unroll
    for (int e = 0; e < V; ++e) v[e] += sm[e] * g - (e == hot ? g : 0.f);
    st<T, V>(dx + i, v);
  }
}

// The same from the logits and the column statistics the forward kernel left
// (maximum, 1 / sum of exponentials) instead of the stored softmax: the softmax
// is rebuilt, rounded to the storage type as the stored one was.  One wave per column.
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void pick_nls_bwd_stats_kernel(int rows, int cols,
                                                                    const typename T::storage* __restrict__ x,
                                                                    const float* __restrict__ stats,
                                                                    const int* __restrict__ idx,
                                                                    const typename T::storage* __restrict__ dout,
                                                                    typename T::storage* dx, int accumulate) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    const float mx = stats[2 * c], inv = stats[2 * c + 1];
    const float g = to_float<T>(dout[c]);
    const int picked = idx[c];
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V], old[V];
      ld<T, V>(x + base + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) old[e] = 0.f;
      if (accumulate) ld<T, V>(dx + base + r, old);
      const int hot = picked - r;
#pragma unroll
      for (int e = 0; e < V; ++e) {
        const float sm = to_float<T>(from_float<T>(softmax_exp<T>(v[e] - mx) * inv));
        v[e] = old[e] + (sm * g - (e == hot ? g : 0.f));
      }
      st<T, V>(dx + base + r, v);
    }
  }
}

}  // namespace
}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_fill(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, void* dst, size_t n, float value) {
  GH_CHECK_ARG(ctx, "ginn_hip_fill: ctx is NULL");
  if (n == 0) return kOk;
  GH_CHECK_ARG(dst, "ginn_hip_fill: dst is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({dst}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (fill_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(static_cast<T::storage*>(dst), n, value)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_copy_2d(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* src, int lds,
                     void* dst, int ldd, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_copy_2d: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_copy_2d: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(src && dst, "ginn_hip_copy_2d: NULL pointer");
  GH_CHECK_ARG(lds >= rows && ldd >= rows, "ginn_hip_copy_2d: leading dimension smaller than rows");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({src, dst}, {static_cast<size_t>(rows), static_cast<size_t>(lds), static_cast<size_t>(ldd)});
  const size_t total = static_cast<size_t>(rows) * cols;
  const unsigned grid = grid_for(vec ? total / 8 : total, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (copy_2d_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(src), lds, static_cast<T::storage*>(dst), ldd, accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_add_n(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, int count, const void* const* host_srcs,
                   void* dst, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_add_n: ctx is NULL");
  GH_CHECK_ARG(count >= 1 && count <= 8, "ginn_hip_add_n: count %d not in 1..8", count);
  if (n == 0) return kOk;
  GH_CHECK_ARG(host_srcs && dst, "ginn_hip_add_n: NULL pointer");
  AddSrcs srcs{};
  for (int k = 0; k < count; ++k) {
    GH_CHECK_ARG(host_srcs[k], "ginn_hip_add_n: source %d is NULL", k);
    srcs.p[k] = host_srcs[k];
  }
  if (dtype == GINN_HIP_I32) {  // two sources per launch
    for (int k = 0; k < count; k += 2) {
      const int rc = launch_int_arith(ctx, kIntAdd, n, 0, host_srcs[k], k + 1 < count ? host_srcs[k + 1] : nullptr,
                                      nullptr, 0, 0, dst, (accumulate || k > 0) ? 1 : 0);
      if (rc != kOk) return rc;
    }
    return kOk;
  }
  GH_HIP(hipSetDevice(ctx->device));
  bool vec = vec8_ok({dst}, {n});
  for (int k = 0; k < count; ++k) vec = vec && vec8_ok({host_srcs[k]}, {});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (add_n_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(n, count, srcs, static_cast<T::storage*>(dst), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_cwise_prod(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* a, const void* b, void* dst,
                        int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_cwise_prod: ctx is NULL");
  if (n == 0) return kOk;
  GH_CHECK_ARG(a && b && dst, "ginn_hip_cwise_prod: NULL pointer");
  if (dtype == GINN_HIP_I32) return launch_int_arith(ctx, kIntMul, n, 0, a, b, nullptr, 0, 0, dst, accumulate);
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({a, b, dst}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (cwise_prod_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      n, static_cast<const T::storage*>(a), static_cast<const T::storage*>(b), static_cast<T::storage*>(dst), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_scale_shift(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, float alpha, float shift, const void* x,
                         void* dst, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_scale_shift: ctx is NULL");
  if (n == 0) return kOk;
  GH_CHECK_ARG(x && dst, "ginn_hip_scale_shift: NULL pointer");
  if (dtype == GINN_HIP_I32)
    return launch_int_arith(ctx, kIntScaleShift, n, 0, x, nullptr, nullptr, static_cast<int>(alpha),
                            static_cast<int>(shift), dst, accumulate);
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({x, dst}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (scale_shift_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      n, alpha, shift, static_cast<const T::storage*>(x), static_cast<T::storage*>(dst), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_col_broadcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, void* dst) {
  GH_CHECK_ARG(ctx, "ginn_hip_col_broadcast: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_col_broadcast: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && dst, "ginn_hip_col_broadcast: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({x, dst}, {static_cast<size_t>(rows)});
  const size_t total = static_cast<size_t>(rows) * cols;
  const unsigned grid = grid_for(vec ? total / 8 : total, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (col_broadcast_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_row_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, void* dst,
                     int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_row_sum: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_row_sum: negative dimension");
  if (rows == 0) return kOk;
  GH_CHECK_ARG(dst && (cols == 0 || x), "ginn_hip_row_sum: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  std::lock_guard<std::mutex> lock(ctx->mutex);
  const bool vec = vec8_ok({x}, {static_cast<size_t>(rows)});
  const rowred::Plan plan = rowred::plan(rows, cols, ctx->num_cus, ctx->workspace_bytes, 1, vec ? 8 : 1);
  GH_CHECK_ARG(plan.chunks >= 1, "ginn_hip_row_sum: workspace too small for %d rows", rows);
  const rowred::Partials room = rowred::take_partials(ctx, static_cast<size_t>(plan.chunks) * rows * sizeof(float));
  float* partial = room.base;
  GH_DISPATCH_DTYPE_V(dtype, vec, (row_sum_partial_kernel<T, V><<<dim3(plan.row_blocks, plan.chunks), rowred::kBlock,
                                                                0, ctx->stream>>>(
      rows, cols, plan.cols_per_chunk, static_cast<const T::storage*>(x), partial)));
  GH_HIP(hipGetLastError());
  return rowred::finish(ctx, {dtype, rows, plan.chunks, accumulate, partial, nullptr, dst, nullptr}, room.deferred);
}

int ginn_hip_sum_all(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* x, float scale, void* dst) {
  GH_CHECK_ARG(ctx, "ginn_hip_sum_all: ctx is NULL");
  GH_CHECK_ARG(dst && (n == 0 || x), "ginn_hip_sum_all: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  if (n <= kSumSmall) {  // a second launch would cost more than the whole sum
    GH_DISPATCH_DTYPE(dtype, (sum_small_kernel<T><<<1, kBlock, 0, ctx->stream>>>(n, static_cast<const T::storage*>(x), scale,
                                                                             static_cast<T::storage*>(dst))));
    GH_HIP(hipGetLastError());
    return kOk;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);
  unsigned blocks = grid_for(n, kBlock * 8, ctx->num_cus);
  if (blocks > 1024) blocks = 1024;
  float* partial = static_cast<float*>(ctx->workspace);
  GH_DISPATCH_DTYPE(dtype, (sum_partial_kernel<T><<<blocks, kBlock, 0, ctx->stream>>>(n, static_cast<const T::storage*>(x), partial)));
  GH_HIP(hipGetLastError());
  GH_DISPATCH_DTYPE(dtype, (sum_fold_kernel<T><<<1, 64, 0, ctx->stream>>>(static_cast<int>(blocks), partial, scale, static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_add_scalar_bcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* src, float scale,
                              void* dst) {
  GH_CHECK_ARG(ctx, "ginn_hip_add_scalar_bcast: ctx is NULL");
  if (n == 0) return kOk;
  GH_CHECK_ARG(src && dst, "ginn_hip_add_scalar_bcast: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({dst}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (add_scalar_bcast_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      n, static_cast<const T::storage*>(src), scale, static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

static int pick_nls_fwd(const char* who, ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x,
                        const int* idx, void* smax, float* stats, void* out) {
  GH_CHECK_ARG(ctx, "%s: ctx is NULL", who);
  GH_CHECK_ARG(rows >= 1 && cols >= 0, "%s: bad dimension", who);
  if (cols == 0) return kOk;
  GH_CHECK_ARG(x && idx && (smax || stats) && out, "%s: NULL pointer", who);
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(cols, kBlock / 64, ctx->num_cus);
  const bool vec = vec8_ok({x, smax}, {static_cast<size_t>(rows)});
  const int vectors = softmax_cols::vectors_for(rows);
  if (vec && vectors) {
    GH_DISPATCH_COLUMN_VECTORS(vectors, {
      GH_DISPATCH_DTYPE(dtype, (pick_nls_fwd_regs_kernel<T, I><<<grid, kBlock, 0, ctx->stream>>>(
          rows, cols, static_cast<const T::storage*>(x), idx, static_cast<T::storage*>(smax), stats,
          static_cast<T::storage*>(out))));
    });
    GH_HIP(hipGetLastError());
    return kOk;
  }
  GH_DISPATCH_DTYPE_V(dtype, vec, (pick_nls_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), idx, static_cast<T::storage*>(smax), stats,
      static_cast<T::storage*>(out))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick_nls_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, const int* idx,
                          void* smax, void* out) {
  GH_CHECK_ARG(smax || cols == 0, "ginn_hip_pick_nls_fwd: NULL pointer");
  return pick_nls_fwd("ginn_hip_pick_nls_fwd", ctx, dtype, rows, cols, x, idx, smax, nullptr, out);
}

int ginn_hip_pick_nls_fwd_stats(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x,
                                const int* idx, float* stats, void* out) {
  GH_CHECK_ARG(stats || cols == 0, "ginn_hip_pick_nls_fwd_stats: NULL pointer");
  return pick_nls_fwd("ginn_hip_pick_nls_fwd_stats", ctx, dtype, rows, cols, x, idx, nullptr, stats, out);
}

int ginn_hip_pick_nls_bwd_stats(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x,
                                const float* stats, const int* idx, const void* dout, void* dx, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_pick_nls_bwd_stats: ctx is NULL");
  GH_CHECK_ARG(rows >= 1 && cols >= 0, "ginn_hip_pick_nls_bwd_stats: bad dimension");
  if (cols == 0) return kOk;
  GH_CHECK_ARG(x && stats && idx && dout && dx, "ginn_hip_pick_nls_bwd_stats: NULL pointer");
  GH_CHECK_ARG(x != dx, "ginn_hip_pick_nls_bwd_stats: dx must not be x");
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({x, dx}, {static_cast<size_t>(rows)});
  const unsigned grid = grid_for(cols, kBlock / 64, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (pick_nls_bwd_stats_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), stats, idx, static_cast<const T::storage*>(dout),
      static_cast<T::storage*>(dx), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

static int pick_nls_bwd(const char* who, ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols,
                        const void* smax, const int* idx, const void* dout, void* dx, int accumulate) {
  GH_CHECK_ARG(ctx, "%s: ctx is NULL", who);
  GH_CHECK_ARG(rows >= 1 && cols >= 0, "%s: bad dimension", who);
  if (cols == 0) return kOk;
  GH_CHECK_ARG(smax && idx && dout && dx, "%s: NULL pointer", who);
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({smax, dx}, {static_cast<size_t>(rows)});
  const size_t total = static_cast<size_t>(rows) * cols;
  const unsigned grid = grid_for(vec ? total / 8 : total, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (pick_nls_bwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(smax), idx, static_cast<const T::storage*>(dout), static_cast<T::storage*>(dx),
      accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick_nls_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* smax,
                          const int* idx, const void* dout, void* dx) {
  return pick_nls_bwd("ginn_hip_pick_nls_bwd", ctx, dtype, rows, cols, smax, idx, dout, dx, 1);
}

int ginn_hip_pick_nls_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* smax,
                                 const int* idx, const void* dout, void* dx) {
  return pick_nls_bwd("ginn_hip_pick_nls_bwd_assign", ctx, dtype, rows, cols, smax, idx, dout, dx, 0);
}

}  // extern "C"
