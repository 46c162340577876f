// Bandwidth-bound companions of the products: stand-alone nonlinearities,
// column-wise softmax, the first half of AffineNode::backward_ and the
// degenerate (m = n = 1) batched product.
#include "common.h"
#include "reduce_rows.h"
#include "kernel_util.h"
#include "vec_access.h"
#include "softmax_cols.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

// ---- elementwise forward / backward ---------------------------------------

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void nonlin_fwd_kernel(
    int act, size_t n, const typename T::storage* __restrict__ x,
    typename T::storage* __restrict__ y) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kBlock * V;
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * V; i < n; i += stride) {
    float v[V];
    ld<T, V>(x + i, v);
    act_forward_n<kFastMath<T>, V>(act, v);
    st<T, V>(y + i, v);
  }
}

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void nonlin_bwd_kernel(
    int act, size_t n, const typename T::storage* __restrict__ dy,
    const typename T::storage* __restrict__ x,
    const typename T::storage* __restrict__ y, typename T::storage* dx,
    int accumulate) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kBlock * V;
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * V; i < n; i += stride) {
    float g[V], xv[V], yv[V], old[V];
    ld<T, V>(dy + i, g);
#pragma unroll
    for (int e = 0; e < V; ++e) xv[e] = yv[e] = old[e] = 0.f;
    if (x) ld<T, V>(x + i, xv);
    if (y) ld<T, V>(y + i, yv);
    if (accumulate) ld<T, V>(dx + i, old);
    act_backward_n<kFastMath<T>, V>(act, xv, yv, g);
#pragma unroll
    for (int e = 0; e < V; ++e) g[e] += old[e];
    st<T, V>(dx + i, g);
  }
}

// ---- column-wise softmax: one wave per column ------------------------------
// ginn/nonlin.h:162-168: subtract the column maximum, exponentiate, divide by
// the column sum.

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void softmax_fwd_kernel(
    int rows, int cols, const typename T::storage* __restrict__ x,
    typename T::storage* __restrict__ y) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const typename T::storage* xc = x + static_cast<size_t>(c) * rows;
    typename T::storage* yc = y + static_cast<size_t>(c) * rows;
    float mx = -INFINITY;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(xc + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) mx = fmaxf(mx, v[e]);
    }
    mx = wave_max(mx);
    float sum = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(xc + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) sum += softmax_exp<T>(v[e] - mx);
    }
    sum = wave_sum(sum);
    const float inv = 1.f / sum;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float v[V];
      ld<T, V>(xc + r, v);
#pragma unroll
      for (int e = 0; e < V; ++e) v[e] = softmax_exp<T>(v[e] - mx) * inv;
      st<T, V>(yc + r, v);
    }
  }
}

// The same with the column in registers (softmax_cols.h); U columns per wave
// and iteration keep more loads in flight when columns are short.  x == y is
// allowed: a wave has read all of its columns before it stores.
template <typename T, int I, int U>
__global__ __launch_bounds__(kBlock) void softmax_fwd_regs_kernel(
    int rows, int cols, const typename T::storage* x, typename T::storage* y) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c0 = wave * U; c0 < cols; c0 += nwaves * U) {
    softmax_cols::Column<T, I> col[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int c = c0 + u < cols ? c0 + u : cols - 1;  // past the end: computed, not stored
      col[u].load(x + static_cast<size_t>(c) * rows, rows, lane);
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      float mx, inv;
      col[u].softmax(mx, inv);
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (c0 + u < cols) col[u].store(y + static_cast<size_t>(c0 + u) * rows, rows, lane);
  }
}

// ginn/nonlin.h:170-188: dx (+)= y * (dy - sum_rows(y * dy)).
template <typename T, int V>
__global__ __launch_bounds__(kBlock) void softmax_bwd_kernel(
    int rows, int cols, const typename T::storage* __restrict__ dy,
    const typename T::storage* __restrict__ y, typename T::storage* dx,
    int accumulate) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float dot = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float yv[V], gv[V];
      ld<T, V>(y + base + r, yv);
      ld<T, V>(dy + base + r, gv);
#pragma unroll
      for (int e = 0; e < V; ++e) dot += yv[e] * gv[e];
    }
    dot = wave_sum(dot);
    for (int r = lane * V; r < rows; r += 64 * V) {
      float yv[V], gv[V], old[V];
      ld<T, V>(y + base + r, yv);
      ld<T, V>(dy + base + r, gv);
#pragma unroll
      for (int e = 0; e < V; ++e) old[e] = 0.f;
      if (accumulate) ld<T, V>(dx + base + r, old);
#pragma unroll
      for (int e = 0; e < V; ++e) gv[e] = yv[e] * (gv[e] - dot) + old[e];
      st<T, V>(dx + base + r, gv);
    }
  }
}

// ---- batched column dot: one wave per column -------------------------------

template <typename T, int V>
__global__ __launch_bounds__(kBlock) void col_dot_kernel(
    int rows, int cols, const typename T::storage* __restrict__ x,
    const typename T::storage* __restrict__ y, float beta,
    typename T::storage* out) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    const size_t base = static_cast<size_t>(c) * rows;
    float dot = 0.f;
    for (int r = lane * V; r < rows; r += 64 * V) {
      float xv[V], yv[V];
      ld<T, V>(x + base + r, xv);
      ld<T, V>(y + base + r, yv);
#pragma unroll
      for (int e = 0; e < V; ++e) dot += xv[e] * yv[e];
    }
    dot = wave_sum(dot);
    if (lane == 0) {
      if (beta != 0.f) dot += beta * to_float<T>(out[c]);
      out[c] = from_float<T>(dot);
    }
  }
}

// ---- AffineNode backward, first half ---------------------------------------
// Pass 1: thread i of a block owns row i of a [256-row x column-chunk] panel:
// consecutive threads touch consecutive addresses of each column.  It writes
// dpre and leaves the fp32 partial row sum of its chunk in `partial`.
// Pass 2 folds the chunks into dbias (storage dtype, accumulating).

template <typename T, int V>
__global__ __launch_bounds__(rowred::kBlock) void affine_bwd_pre_kernel(
    int act, int m, int n, int cols_per_chunk,
    const typename T::storage* __restrict__ dy,
    const typename T::storage* __restrict__ y,
    const typename T::storage* __restrict__ pre,
    typename T::storage* __restrict__ dpre, float* __restrict__ partial) {
  __shared__ float red[rowred::kSlices * V * 64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int row = (blockIdx.x * rowred::kRowsPerBlock + tx) * V;
  const int c0 = blockIdx.y * cols_per_chunk;
  int c1 = c0 + cols_per_chunk;
  if (c1 > n) c1 = n;
  float sum[V];
#pragma unroll
  for (int e = 0; e < V; ++e) sum[e] = 0.f;
  if (row < m) {
    // Four columns per step, all their loads issued before the first use: a
    // block of a small matrix has only a few columns, and one at a time would
    // pay a memory latency for each.
    constexpr int U = 4;
    for (int c = c0 + ty; c < c1; c += U * rowred::kSlices) {
      float g[U][V], xv[U][V], yv[U][V];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cu = c + u * rowred::kSlices;
#pragma unroll
        for (int e = 0; e < V; ++e) g[u][e] = xv[u][e] = yv[u][e] = 0.f;
        if (cu < c1) {
          const size_t i = static_cast<size_t>(cu) * m + row;
          ld<T, V>(dy + i, g[u]);
          if (act != GINN_HIP_ACT_IDENTITY) {
            if (pre) ld<T, V>(pre + i, xv[u]);
            if (y) ld<T, V>(y + i, yv[u]);
          }
        }
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cu = c + u * rowred::kSlices;
        if (cu < c1) {
          if (act != GINN_HIP_ACT_IDENTITY) {
            act_backward_n<kFastMath<T>, V>(act, xv[u], yv[u], g[u]);
            // The row sum uses the value as stored, i.e. what the products see.
#pragma unroll
            for (int e = 0; e < V; ++e) g[u][e] = to_float<T>(from_float<T>(g[u][e]));
            st<T, V>(dpre + static_cast<size_t>(cu) * m + row, g[u]);
          }
#pragma unroll
          for (int e = 0; e < V; ++e) sum[e] += g[u][e];
        }
      }
    }
  }
  if (!partial) return;
  rowred::combine_v<V>(sum, red);
  if (ty == 0 && row < m) {
#pragma unroll
    for (int e = 0; e < V; ++e) partial[static_cast<size_t>(blockIdx.y) * m + row + e] = sum[e];
  }
}

}  // namespace

int launch_softmax_fwd(ginn_hip_ctx* ctx, int dtype, int rows, int cols,
                       const void* x, void* y) {
  if (rows == 0 || cols == 0) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({x, y}, {static_cast<size_t>(rows)});
  const int vectors = softmax_cols::vectors_for(rows);
  if (vec && vectors) {
    GH_DISPATCH_COLUMN_VECTORS(vectors, {
      constexpr int U = I == 1 ? 4 : I == 2 ? 2 : 1;
      const unsigned grid = grid_for((cols + U - 1) / U, kBlock / 64, ctx->num_cus);
      GH_DISPATCH_DTYPE(dtype, (softmax_fwd_regs_kernel<T, I, U><<<grid, kBlock, 0, ctx->stream>>>(
          rows, cols, static_cast<const T::storage*>(x), static_cast<T::storage*>(y))));
    });
    GH_HIP(hipGetLastError());
    return kOk;
  }
  const unsigned grid = grid_for(cols, kBlock / 64, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (softmax_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), static_cast<T::storage*>(y))));
  GH_HIP(hipGetLastError());
  return kOk;
}

}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_nonlin_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int rows, int cols, const void* x,
                        void* y) {
  GH_CHECK_ARG(ctx, "ginn_hip_nonlin_fwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_nonlin_fwd: negative dimension");
  GH_CHECK_ARG(act >= GINN_HIP_ACT_IDENTITY && act <= GINN_HIP_ACT_SQRT,
               "ginn_hip_nonlin_fwd: unknown activation %d", act);
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && y, "ginn_hip_nonlin_fwd: NULL pointer");
  if (act == GINN_HIP_ACT_SOFTMAX) return launch_softmax_fwd(ctx, dtype, rows, cols, x, y);
  GH_HIP(hipSetDevice(ctx->device));
  const size_t n = static_cast<size_t>(rows) * cols;
  const bool vec = vec8_ok({x, y}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE_V(dtype, vec, (nonlin_fwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      act, n, static_cast<const T::storage*>(x), static_cast<T::storage*>(y))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_nonlin_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int rows, int cols, const void* dy,
                        const void* x, const void* y, void* dx,
                        int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_nonlin_bwd: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_nonlin_bwd: negative dimension");
  GH_CHECK_ARG(act >= GINN_HIP_ACT_IDENTITY && act <= GINN_HIP_ACT_SQRT,
               "ginn_hip_nonlin_bwd: unknown activation %d", act);
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(dy && dx, "ginn_hip_nonlin_bwd: NULL pointer");
  const bool needs_x = act_backward_requires_input(act) && act != GINN_HIP_ACT_SOFTMAX;
  const bool needs_y = act == GINN_HIP_ACT_TANH || act == GINN_HIP_ACT_RELU ||
                       act == GINN_HIP_ACT_SIGMOID || act == GINN_HIP_ACT_SOFTMAX ||
                       act == GINN_HIP_ACT_SQRT;
  GH_CHECK_ARG(!needs_x || x, "ginn_hip_nonlin_bwd: this activation needs x");
  GH_CHECK_ARG(!needs_y || y, "ginn_hip_nonlin_bwd: this activation needs y");
  GH_HIP(hipSetDevice(ctx->device));
  if (act == GINN_HIP_ACT_SOFTMAX) {
    const unsigned grid = grid_for(cols, kBlock / 64, ctx->num_cus);
    const bool vec = vec8_ok({dy, y, dx}, {static_cast<size_t>(rows)});
    GH_DISPATCH_DTYPE_V(dtype, vec, (softmax_bwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
        rows, cols, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(y),
        static_cast<T::storage*>(dx), accumulate)));
  } else {
    const size_t n = static_cast<size_t>(rows) * cols;
    const bool vec = vec8_ok({dy, x, y, dx}, {n});
    const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
    GH_DISPATCH_DTYPE_V(dtype, vec, (nonlin_bwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
        act, n, static_cast<const T::storage*>(dy), static_cast<const T::storage*>(x),
        static_cast<const T::storage*>(y), static_cast<T::storage*>(dx), accumulate)));
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_col_dot_batched(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                             int cols, const void* x, const void* y, float beta,
                             void* out) {
  GH_CHECK_ARG(ctx, "ginn_hip_col_dot_batched: ctx is NULL");
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_col_dot_batched: negative dimension");
  if (cols == 0) return kOk;
  GH_CHECK_ARG(out && (rows == 0 || (x && y)), "ginn_hip_col_dot_batched: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(cols, kBlock / 64, ctx->num_cus);
  const bool vec = vec8_ok({x, y}, {static_cast<size_t>(rows)});
  GH_DISPATCH_DTYPE_V(dtype, vec, (col_dot_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
      rows, cols, static_cast<const T::storage*>(x), static_cast<const T::storage*>(y), beta,
      static_cast<T::storage*>(out))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_affine_bwd_pre(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                            ginn_hip_act act, int m, int n, const void* dY,
                            const void* Y, const void* pre, void* dpre,
                            void* dbias) {
  GH_CHECK_ARG(ctx, "ginn_hip_affine_bwd_pre: ctx is NULL");
  GH_CHECK_ARG(m >= 0 && n >= 0, "ginn_hip_affine_bwd_pre: negative dimension");
  GH_CHECK_ARG(act >= GINN_HIP_ACT_IDENTITY && act <= GINN_HIP_ACT_SOFTMAX,
               "ginn_hip_affine_bwd_pre: activation %d cannot be carried by an Affine", act);
  if (m == 0 || n == 0) return kOk;
  GH_CHECK_ARG(dY, "ginn_hip_affine_bwd_pre: dY is NULL");
  const bool identity = act == GINN_HIP_ACT_IDENTITY;
  GH_CHECK_ARG(identity || dpre, "ginn_hip_affine_bwd_pre: dpre is NULL");
  GH_CHECK_ARG(identity || act_backward_requires_input(act) ? true : Y != nullptr,
               "ginn_hip_affine_bwd_pre: this activation needs Y");
  GH_CHECK_ARG(!act_backward_requires_input(act) || act == GINN_HIP_ACT_SOFTMAX || pre,
               "ginn_hip_affine_bwd_pre: this activation needs the pre-activation");
  GH_CHECK_ARG(act != GINN_HIP_ACT_SOFTMAX || Y, "ginn_hip_affine_bwd_pre: SOFTMAX needs Y");
  if (identity && !dbias) return kOk;
  GH_HIP(hipSetDevice(ctx->device));

  const void* bias_src = dY;  // matrix whose rows are summed into dbias
  int bias_act = act;
  if (act == GINN_HIP_ACT_SOFTMAX) {
    // dpre = y * (dy - colsum(y * dy)): column-wise, its own kernel; the row
    // sums are then taken over dpre like for the identity.
    const unsigned grid = grid_for(n, kBlock / 64, ctx->num_cus);
    const bool vec = vec8_ok({dY, Y, dpre}, {static_cast<size_t>(m)});
    GH_DISPATCH_DTYPE_V(dtype, vec, (softmax_bwd_kernel<T, V><<<grid, kBlock, 0, ctx->stream>>>(
        m, n, static_cast<const T::storage*>(dY), static_cast<const T::storage*>(Y),
        static_cast<T::storage*>(dpre), 0)));
    GH_HIP(hipGetLastError());
    if (!dbias) return kOk;
    bias_src = dpre;
    bias_act = GINN_HIP_ACT_IDENTITY;
  }

  // The kernel reads what the derivative is written in: the pre-activation (GELU, GELU2, LOG) or the
  // output (the others), not both.
  if (bias_act != GINN_HIP_ACT_IDENTITY) {
    if (act_backward_requires_input(bias_act)) Y = nullptr;
    else pre = nullptr;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);
  const bool vec = vec8_ok({bias_src, Y, pre, dpre}, {static_cast<size_t>(m)});
  const rowred::Plan plan = rowred::plan(m, n, ctx->num_cus, ctx->workspace_bytes, 1, vec ? 8 : 1);
  GH_CHECK_ARG(plan.chunks >= 1, "ginn_hip_affine_bwd_pre: workspace too small for m=%d", m);
  rowred::Partials room{nullptr, false};
  if (dbias) room = rowred::take_partials(ctx, static_cast<size_t>(plan.chunks) * m * sizeof(float));
  float* partial = room.base;
  const dim3 grid(plan.row_blocks, plan.chunks);
  GH_DISPATCH_DTYPE_V(dtype, vec, (affine_bwd_pre_kernel<T, V><<<grid, rowred::kBlock, 0, ctx->stream>>>(
      bias_act, m, n, plan.cols_per_chunk, static_cast<const T::storage*>(bias_src),
      static_cast<const T::storage*>(Y), static_cast<const T::storage*>(pre),
      static_cast<T::storage*>(dpre), partial)));
  GH_HIP(hipGetLastError());
  if (dbias) return rowred::finish(ctx, {dtype, m, plan.chunks, 1, partial, nullptr, dbias, nullptr}, room.deferred);
  return kOk;
}

}  // extern "C"
