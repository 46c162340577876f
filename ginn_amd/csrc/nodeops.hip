// Device side of the remaining element-wise, selection, gather / scatter and
// reduction nodes that surround the product path in the reference's graphs
// (ginn/node/common.h, select.h, compare.h, pick.h, reduce.h, layout.h,
// inplace.h, ginn/util/amax.h, Tensor::set_random).  The reference evaluates
// them as Eigen expressions, thrust gathers and two hand-written kernels
// (Stack); here each is one small kernel, bound by memory or by launch cost.
#include "common.h"
#include "kernel_util.h"
#include "vec_access.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

#define GH_GRID_STRIDE_V(i, n, V)                                              \
  for (size_t i = (blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x) * (V), \
              stride__ = static_cast<size_t>(gridDim.x) * kBlock * (V);        \
       i < (n); i += stride__)
#define GH_GRID_STRIDE(i, n) GH_GRID_STRIDE_V(i, n, 1)

// ---------------------------------------------------------------------------
// Two- and three-operand element-wise forms
// ---------------------------------------------------------------------------

template <typename T, int V, int OP>
__global__ __launch_bounds__(kBlock) void elementwise_kernel(size_t n, const typename T::storage* a,
                                                             const typename T::storage* b,
                                                             const typename T::storage* c,
                                                             typename T::storage* dst, int accumulate) {
  GH_GRID_STRIDE_V(i, n, V) {
    float x[V], y[V], z[V], old[V];
    ld<T, V>(a + i, x);
    ld<T, V>(b + i, y);
#pragma unroll
    for (int e = 0; e < V; ++e) z[e] = old[e] = 0.f;
    if (OP == GINN_HIP_EW_EQ_MUL || OP == GINN_HIP_EW_DIV_MUL) ld<T, V>(c + i, z);
    if (accumulate) ld<T, V>(dst + i, old);
#pragma unroll
    for (int e = 0; e < V; ++e) {
      float r;
      if (OP == GINN_HIP_EW_SUB) r = x[e] - y[e];
      else if (OP == GINN_HIP_EW_MAX) r = fmaxf(x[e], y[e]);
      else if (OP == GINN_HIP_EW_EQ_MUL) r = y[e] == z[e] ? x[e] : 0.f;
      else r = x[e] * (y[e] / z[e]);
      x[e] = r + old[e];
    }
    st<T, V>(dst + i, x);
  }
}

// dst (+)= x * mask * scale, mask one byte per element.
template <typename T>
__global__ __launch_bounds__(kBlock) void mask_scale_kernel(size_t n, float scale, const typename T::storage* x,
                                                            const uint8_t* __restrict__ mask,
                                                            typename T::storage* dst, int accumulate) {
  GH_GRID_STRIDE(i, n) {
    float v = mask[i] ? to_float<T>(x[i]) * scale : 0.f;
    if (accumulate) v += to_float<T>(dst[i]);
    dst[i] = from_float<T>(v);
  }
}

// ---------------------------------------------------------------------------
// Random numbers: element i of a fill with seed s is a function of (s, i)
// alone (SplitMix64 of the pair), so a fill does not depend on the launch
// geometry and two fills with different seeds are independent streams.
// ---------------------------------------------------------------------------

__device__ __forceinline__ float uniform01(uint64_t seed, size_t i) {
  uint64_t z = seed + 0x9e3779b97f4a7c15ull * (static_cast<uint64_t>(i) + 1);
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  z ^= z >> 31;
  return static_cast<float>(z >> 40) * (1.0f / 16777216.0f);  // 24 bits: exact in fp32, < 1
}

template <typename T>
__global__ __launch_bounds__(kBlock) void fill_uniform_kernel(size_t n, uint64_t seed, float lo, float hi,
                                                              typename T::storage* dst) {
  GH_GRID_STRIDE(i, n) dst[i] = from_float<T>(lo + (hi - lo) * uniform01(seed, i));
}

__global__ __launch_bounds__(kBlock) void dropout_mask_kernel(size_t n, float p, uint64_t seed, uint8_t* mask) {
  GH_GRID_STRIDE(i, n) mask[i] = uniform01(seed, i) >= p ? 1 : 0;
}

// ---------------------------------------------------------------------------
// Select, Mask, LessThan
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kBlock) void select_kernel(size_t n, const uint8_t* __restrict__ cond,
                                                        const typename T::storage* a, int a_scalar,
                                                        const typename T::storage* b, int b_scalar,
                                                        typename T::storage* dst) {
  GH_GRID_STRIDE(i, n) dst[i] = cond[i] ? a[a_scalar ? 0 : i] : b[b_scalar ? 0 : i];
}

// dst[i] += dy[i] where (cond[i] != 0) == want.
template <typename T>
__global__ __launch_bounds__(kBlock) void select_bwd_kernel(size_t n, const uint8_t* __restrict__ cond, int want,
                                                            const typename T::storage* __restrict__ dy,
                                                            typename T::storage* dst) {
  GH_GRID_STRIDE(i, n) {
    if ((cond[i] != 0) == (want != 0)) dst[i] = from_float<T>(to_float<T>(dst[i]) + to_float<T>(dy[i]));
  }
}
// The same summed into one element (a branch that is a single value): one block.
template <typename T>
__global__ __launch_bounds__(kBlock) void select_bwd_scalar_kernel(size_t n, const uint8_t* __restrict__ cond,
                                                                   int want,
                                                                   const typename T::storage* __restrict__ dy,
                                                                   typename T::storage* dst) {
  __shared__ float ws[kBlock / 64];
  float s = 0.f;
  for (size_t i = threadIdx.x; i < n; i += kBlock)
    if ((cond[i] != 0) == (want != 0)) s += to_float<T>(dy[i]);
  s = wave_sum(s);
  if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = s;
  __syncthreads();
  if (threadIdx.x == 0) {
    float t = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) t += ws[w];
    dst[0] = from_float<T>(to_float<T>(dst[0]) + t);
  }
}

// dst (+)= mask[i % mask_size] != 0 ? x[i] : value.
template <typename T>
__global__ __launch_bounds__(kBlock) void mask_select_kernel(size_t mask_size, size_t n,
                                                             const typename T::storage* __restrict__ mask,
                                                             float value, const typename T::storage* x,
                                                             typename T::storage* dst, int accumulate) {
  GH_GRID_STRIDE(i, n) {
    float v = to_float<T>(mask[i % mask_size]) != 0.f ? to_float<T>(x[i]) : value;
    if (accumulate) v += to_float<T>(dst[i]);
    dst[i] = from_float<T>(v);
  }
}

template <typename T>
__global__ __launch_bounds__(kBlock) void less_than_kernel(size_t n, const typename T::storage* __restrict__ a,
                                                           const typename T::storage* __restrict__ b,
                                                           uint8_t* out) {
  GH_GRID_STRIDE(i, n) out[i] = to_float<T>(a[i]) < to_float<T>(b[i]) ? 1 : 0;
}
__global__ __launch_bounds__(kBlock) void less_than_int_kernel(size_t n, const int* __restrict__ a,
                                                               const int* __restrict__ b, uint8_t* out) {
  GH_GRID_STRIDE(i, n) out[i] = a[i] < b[i] ? 1 : 0;
}

// ---------------------------------------------------------------------------
// Pick family
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kBlock) void pick_kernel(int rows, int cols, const typename T::storage* __restrict__ x,
                                                      const int* __restrict__ idx, typename T::storage* out) {
  GH_GRID_STRIDE(c, static_cast<size_t>(cols)) {
    const int r = idx[c];
    // an index outside the column picks nothing: NaN shows it
    out[c] = (r >= 0 && r < rows) ? x[c * rows + r] : from_float<T>(NAN);
  }
}
template <typename T>
__global__ __launch_bounds__(kBlock) void pick_bwd_kernel(int rows, int cols, const int* __restrict__ idx,
                                                          const typename T::storage* __restrict__ dout, float sign,
                                                          typename T::storage* dx) {
  GH_GRID_STRIDE(c, static_cast<size_t>(cols)) {
    const int r = idx[c];
    if (r >= 0 && r < rows) {
      const size_t at = c * rows + r;
      dx[at] = from_float<T>(to_float<T>(dx[at]) + sign * to_float<T>(dout[c]));
    }
  }
}

// sigm = sigmoid(x); out = -(idx ? log(sigm) : log(1 - sigm)), elementwise
// (ginn/node/pick.h:250-272), from the stored (rounded) sigmoid as there.
template <typename T>
__global__ __launch_bounds__(kBlock) void pick_nlsig_fwd_kernel(size_t n, const typename T::storage* __restrict__ x,
                                                                const int* __restrict__ idx,
                                                                typename T::storage* sigm,
                                                                typename T::storage* out) {
  GH_GRID_STRIDE(i, n) {
    const typename T::storage s_st = from_float<T>(act_forward_c<false, GINN_HIP_ACT_SIGMOID>(to_float<T>(x[i])));
    sigm[i] = s_st;
    const float s = to_float<T>(s_st);
    out[i] = from_float<T>(-(idx[i] ? logf(s) : logf(1.f - s)));
  }
}
template <typename T>
__global__ __launch_bounds__(kBlock) void pick_nlsig_bwd_kernel(size_t n,
                                                                const typename T::storage* __restrict__ sigm,
                                                                const int* __restrict__ idx,
                                                                const typename T::storage* __restrict__ dout,
                                                                typename T::storage* dx) {
  GH_GRID_STRIDE(i, n) {
    const float g = (to_float<T>(sigm[i]) - static_cast<float>(idx[i])) * to_float<T>(dout[i]);
    dx[i] = from_float<T>(to_float<T>(dx[i]) + g);
  }
}

// ---------------------------------------------------------------------------
// Reductions over chosen axes; scalar variance
// ---------------------------------------------------------------------------

struct AxisDesc {
  int rank;
  long long dim[8];
  long long out_stride[8];  // stride of the axis in the reduced tensor, 0 for a summed axis
  long long n_in, n_out;
};

// One thread per output element, looping over the summed axes (small tensors:
// the reference uses it for statistics and attention-free pooling).
template <typename T>
__global__ __launch_bounds__(kBlock) void axis_sum_kernel(AxisDesc d, const typename T::storage* __restrict__ x,
                                                          typename T::storage* dst) {
  GH_GRID_STRIDE(o, static_cast<size_t>(d.n_out)) {
    // coordinates of the output element along the kept axes
    long long base = 0, in_stride = 1, rem = static_cast<long long>(o);
    long long red_dim[8], red_stride[8];
    int nred = 0;
    for (int a = 0; a < d.rank; ++a) {
      if (d.out_stride[a] == 0) {
        red_dim[nred] = d.dim[a];
        red_stride[nred] = in_stride;
        ++nred;
      } else {
        base += (rem % d.dim[a]) * in_stride;
        rem /= d.dim[a];
      }
      in_stride *= d.dim[a];
    }
    long long total = 1;
    for (int r = 0; r < nred; ++r) total *= red_dim[r];
    float s = 0.f;
    for (long long t = 0; t < total; ++t) {
      long long off = base, q = t;
      for (int r = 0; r < nred; ++r) {
        off += (q % red_dim[r]) * red_stride[r];
        q /= red_dim[r];
      }
      s += to_float<T>(x[off]);
    }
    dst[o] = from_float<T>(s);
  }
}
// dx[i] += dy[projection of i onto the kept axes].
template <typename T>
__global__ __launch_bounds__(kBlock) void axis_sum_bwd_kernel(AxisDesc d, const typename T::storage* __restrict__ dy,
                                                              typename T::storage* dx) {
  GH_GRID_STRIDE(i, static_cast<size_t>(d.n_in)) {
    long long rem = static_cast<long long>(i), o = 0;
    for (int a = 0; a < d.rank; ++a) {
      o += (rem % d.dim[a]) * d.out_stride[a];
      rem /= d.dim[a];
    }
    dx[i] = from_float<T>(to_float<T>(dx[i]) + to_float<T>(dy[o]));
  }
}

// mean and biased variance of n values, one block, two passes (ginn/node/reduce.h:164-177).
template <typename T>
__global__ __launch_bounds__(kBlock) void variance_fwd_kernel(size_t n, const typename T::storage* __restrict__ x,
                                                              typename T::storage* mean_out,
                                                              typename T::storage* var_out) {
  __shared__ float ws[kBlock / 64];
  __shared__ float mean_s;
  auto block_sum = [&](float s) {
    s = wave_sum(s);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) ws[threadIdx.x >> 6] = s;
    __syncthreads();
    float t = 0.f;
    for (int w = 0; w < kBlock / 64; ++w) t += ws[w];
    return t;
  };
  float s = 0.f;
  for (size_t i = threadIdx.x; i < n; i += kBlock) s += to_float<T>(x[i]);
  const float total = block_sum(s);
  if (threadIdx.x == 0) {
    // the mean is kept as a tensor of the node's scalar type, as in the reference
    const typename T::storage m = from_float<T>(total / static_cast<float>(n));
    mean_out[0] = m;
    mean_s = to_float<T>(m);
  }
  __syncthreads();
  const float mean = mean_s;
  float q = 0.f;
  for (size_t i = threadIdx.x; i < n; i += kBlock) {
    const float dlt = to_float<T>(x[i]) - mean;
    q += dlt * dlt;
  }
  const float qsum = block_sum(q);
  if (threadIdx.x == 0) var_out[0] = from_float<T>(qsum / static_cast<float>(n));
}
template <typename T>
__global__ __launch_bounds__(kBlock) void variance_bwd_kernel(size_t n, const typename T::storage* __restrict__ x,
                                                              const typename T::storage* __restrict__ mean,
                                                              const typename T::storage* __restrict__ dvar,
                                                              typename T::storage* dx) {
  const float m = to_float<T>(mean[0]), g = to_float<T>(dvar[0]) * (2.f / static_cast<float>(n));
  GH_GRID_STRIDE(i, n) dx[i] = from_float<T>(to_float<T>(dx[i]) + (to_float<T>(x[i]) - m) * g);
}

// ---------------------------------------------------------------------------
// Stack: `count` arrays of sz elements each, found through a pointer table,
// into one contiguous tensor, and its backward scatter-add
// (ginn/node/layout.h:324-348).  A table may name one array several times
// (the same embedding looked up twice), so the backward pass adds atomically.
// ---------------------------------------------------------------------------

template <typename S>
__global__ __launch_bounds__(kBlock) void stack_kernel(size_t sz, size_t count, const S* const* __restrict__ srcs,
                                                       S* dst) {
  const size_t total = sz * count;
  GH_GRID_STRIDE(i, total) dst[i] = srcs[i / sz][i % sz];
}

__device__ __forceinline__ void atomic_add_elem(float* p, float v) { atomicAdd(p, v); }
// A 16-bit element is updated through a compare-and-swap on the aligned
// 32-bit word that holds it.
template <typename T>
__device__ __forceinline__ void atomic_add_elem16(uint16_t* p, float v) {
  const uintptr_t addr = reinterpret_cast<uintptr_t>(p);
  unsigned int* word = reinterpret_cast<unsigned int*>(addr & ~uintptr_t(3));
  const bool high = (addr & 2) != 0;
  unsigned int seen = *word, want;
  do {
    const uint16_t cur = high ? static_cast<uint16_t>(seen >> 16) : static_cast<uint16_t>(seen & 0xffffu);
    const uint16_t upd = from_float<T>(to_float<T>(cur) + v);
    want = high ? ((seen & 0x0000ffffu) | (static_cast<unsigned int>(upd) << 16))
                : ((seen & 0xffff0000u) | upd);
    const unsigned int prev = atomicCAS(word, seen, want);
    if (prev == seen) break;
    seen = prev;
  } while (true);
}

template <typename T>
__global__ __launch_bounds__(kBlock) void stack_bwd_kernel(size_t sz, size_t count,
                                                           typename T::storage* const* __restrict__ dsts,
                                                           const typename T::storage* __restrict__ src) {
  const size_t total = sz * count;
  GH_GRID_STRIDE(i, total) {
    typename T::storage* d = dsts[i / sz];
    if (!d) continue;  // an input without gradient
    if constexpr (sizeof(typename T::storage) == 4) atomic_add_elem(d + i % sz, src[i]);
    else atomic_add_elem16<T>(d + i % sz, to_float<T>(src[i]));
  }
}

// ---------------------------------------------------------------------------
// argmax along the middle axis of [inner, len, outer]; first maximum wins
// (std::max_element, ginn/util/amax.h:28-66).
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kBlock) void argmax_kernel(size_t inner, size_t len, size_t outer,
                                                        const typename T::storage* __restrict__ x,
                                                        long long* out) {
  GH_GRID_STRIDE(o, inner * outer) {
    const size_t in = o % inner, ou = o / inner;
    const typename T::storage* col = x + ou * len * inner + in;
    float best = to_float<T>(col[0]);
    long long at = 0;
    for (size_t l = 1; l < len; ++l) {
      const float v = to_float<T>(col[l * inner]);
      if (v > best) {
        best = v;
        at = static_cast<long long>(l);
      }
    }
    out[o] = at;
  }
}

// ---------------------------------------------------------------------------
// Row broadcast and its backward (column sums)
// ---------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(kBlock) void row_broadcast_kernel(int rows, size_t n,
                                                               const typename T::storage* __restrict__ x,
                                                               typename T::storage* dst) {
  GH_GRID_STRIDE(i, n) dst[i] = x[i / rows];
}
// dst[c] (+)= sum_r x[r, c]: one wave per column.
template <typename T>
__global__ __launch_bounds__(kBlock) void col_sum_kernel(int rows, int cols,
                                                         const typename T::storage* __restrict__ x,
                                                         typename T::storage* dst, int accumulate) {
  const int lane = threadIdx.x & 63;
  const int wave = blockIdx.x * (kBlock / 64) + (threadIdx.x >> 6);
  const int nwaves = gridDim.x * (kBlock / 64);
  for (int c = wave; c < cols; c += nwaves) {
    float s = 0.f;
    for (int r = lane; r < rows; r += 64) s += to_float<T>(x[static_cast<size_t>(c) * rows + r]);
    s = wave_sum(s);
    if (lane == 0) dst[c] = from_float<T>(s + (accumulate ? to_float<T>(dst[c]) : 0.f));
  }
}

}  // namespace
}  // namespace ginn_hip

using namespace ginn_hip;

#define GH_ENTER(name, ctx)                                                    \
  GH_CHECK_ARG(ctx, name ": ctx is NULL");                                     \
  GH_CHECK_ARG(dtype_valid(dtype), name ": unknown dtype %d", dtype)
// The same for entry points that also take 32-bit integers.
#define GH_ENTER_OR_INT(name, ctx)                                             \
  GH_CHECK_ARG(ctx, name ": ctx is NULL");                                     \
  GH_CHECK_ARG(dtype_valid(dtype) || dtype == GINN_HIP_I32, name ": unknown dtype %d", dtype)

extern "C" {

int ginn_hip_elementwise(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, ginn_hip_ew_op op, size_t n, const void* a,
                         const void* b, const void* c, void* dst, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_elementwise: ctx is NULL");
  GH_CHECK_ARG(dtype_valid(dtype) || dtype == GINN_HIP_I32, "ginn_hip_elementwise: unknown dtype %d", dtype);
  GH_CHECK_ARG(op >= GINN_HIP_EW_SUB && op <= GINN_HIP_EW_DIV_MUL, "ginn_hip_elementwise: unknown op %d", op);
  if (n == 0) return kOk;
  const bool three = op == GINN_HIP_EW_EQ_MUL || op == GINN_HIP_EW_DIV_MUL;
  GH_CHECK_ARG(a && b && dst && (!three || c), "ginn_hip_elementwise: NULL operand");
  if (dtype == GINN_HIP_I32) {
    GH_CHECK_ARG(!three, "ginn_hip_elementwise: operation %d has no integer form", op);
    return launch_int_arith(ctx, op == GINN_HIP_EW_SUB ? kIntSub : kIntMax, n, 0, a, b, nullptr, 0, 0, dst,
                            accumulate);
  }
  GH_HIP(hipSetDevice(ctx->device));
  const bool vec = vec8_ok({a, b, c, dst}, {n});
  const unsigned grid = grid_for(vec ? n / 8 : n, kBlock, ctx->num_cus);
#define GH_EW(OPC)                                                                                         \
  GH_DISPATCH_DTYPE_V(dtype, vec,                                                                          \
                      (elementwise_kernel<T, V, OPC><<<grid, kBlock, 0, ctx->stream>>>(                    \
                          n, static_cast<const T::storage*>(a), static_cast<const T::storage*>(b),         \
                          static_cast<const T::storage*>(c), static_cast<T::storage*>(dst), accumulate)))
  switch (op) {
    case GINN_HIP_EW_SUB: GH_EW(GINN_HIP_EW_SUB); break;
    case GINN_HIP_EW_MAX: GH_EW(GINN_HIP_EW_MAX); break;
    case GINN_HIP_EW_EQ_MUL: GH_EW(GINN_HIP_EW_EQ_MUL); break;
    default: GH_EW(GINN_HIP_EW_DIV_MUL); break;
  }
#undef GH_EW
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_mask_scale(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, float scale, const void* x,
                        const unsigned char* mask, void* dst, int accumulate) {
  GH_ENTER("ginn_hip_mask_scale", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(x && mask && dst, "ginn_hip_mask_scale: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (mask_scale_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               n, scale, static_cast<const T::storage*>(x), mask, static_cast<T::storage*>(dst),
                               accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_fill_uniform(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, unsigned long long seed, float lo,
                          float hi, void* dst) {
  GH_ENTER("ginn_hip_fill_uniform", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(dst, "ginn_hip_fill_uniform: dst is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (fill_uniform_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(n, seed, lo, hi,
                                                                                     static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_dropout_mask(ginn_hip_ctx* ctx, size_t n, float p, unsigned long long seed, unsigned char* mask) {
  GH_CHECK_ARG(ctx, "ginn_hip_dropout_mask: ctx is NULL");
  GH_CHECK_ARG(p >= 0.f && p <= 1.f, "ginn_hip_dropout_mask: probability %g is not in [0, 1]", p);
  if (n == 0) return kOk;
  GH_CHECK_ARG(mask, "ginn_hip_dropout_mask: mask is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  dropout_mask_kernel<<<grid_for(n, kBlock, ctx->num_cus), kBlock, 0, ctx->stream>>>(n, p, seed, mask);
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_select(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const unsigned char* cond, const void* a,
                    int a_is_scalar, const void* b, int b_is_scalar, void* dst) {
  GH_ENTER_OR_INT("ginn_hip_select", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(cond && a && b && dst, "ginn_hip_select: NULL operand");
  if (dtype == GINN_HIP_I32) return launch_int_select(ctx, n, cond, a, a_is_scalar, b, b_is_scalar, dst);
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (select_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               n, cond, static_cast<const T::storage*>(a), a_is_scalar,
                               static_cast<const T::storage*>(b), b_is_scalar, static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_select_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const unsigned char* cond, int want,
                        const void* dy, void* dst, int dst_is_scalar) {
  GH_ENTER("ginn_hip_select_bwd", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(cond && dy && dst, "ginn_hip_select_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  if (dst_is_scalar) {
    GH_DISPATCH_DTYPE(dtype, (select_bwd_scalar_kernel<T><<<1, kBlock, 0, ctx->stream>>>(
                                 n, cond, want, static_cast<const T::storage*>(dy), static_cast<T::storage*>(dst))));
  } else {
    const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
    GH_DISPATCH_DTYPE(dtype, (select_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                                 n, cond, want, static_cast<const T::storage*>(dy), static_cast<T::storage*>(dst))));
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_mask_select(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t mask_size, size_t batch, const void* mask,
                         float value, const void* x, void* dst, int accumulate) {
  GH_ENTER_OR_INT("ginn_hip_mask_select", ctx);
  const size_t n = mask_size * batch;
  if (n == 0) return kOk;
  GH_CHECK_ARG(mask && x && dst, "ginn_hip_mask_select: NULL operand");
  if (dtype == GINN_HIP_I32) {
    GH_CHECK_ARG(!accumulate, "ginn_hip_mask_select: 32-bit integers have no gradient to accumulate");
    return launch_int_mask(ctx, mask_size, n, mask, static_cast<int>(value), x, dst);
  }
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (mask_select_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               mask_size, n, static_cast<const T::storage*>(mask), value,
                               static_cast<const T::storage*>(x), static_cast<T::storage*>(dst), accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_less_than(ginn_hip_ctx* ctx, int dtype, size_t n, const void* a, const void* b, unsigned char* out) {
  GH_CHECK_ARG(ctx, "ginn_hip_less_than: ctx is NULL");
  GH_CHECK_ARG(dtype_valid(dtype) || dtype == GINN_HIP_I32, "ginn_hip_less_than: unknown dtype %d", dtype);
  if (n == 0) return kOk;
  GH_CHECK_ARG(a && b && out, "ginn_hip_less_than: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  if (dtype == GINN_HIP_I32) {
    less_than_int_kernel<<<grid, kBlock, 0, ctx->stream>>>(n, static_cast<const int*>(a), static_cast<const int*>(b),
                                                           out);
  } else {
    GH_DISPATCH_DTYPE(dtype, (less_than_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                                 n, static_cast<const T::storage*>(a), static_cast<const T::storage*>(b), out)));
  }
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, const int* idx,
                  void* out) {
  GH_ENTER("ginn_hip_pick", ctx);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_pick: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && idx && out, "ginn_hip_pick: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(cols, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (pick_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               rows, cols, static_cast<const T::storage*>(x), idx, static_cast<T::storage*>(out))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const int* idx, const void* dout,
                      float sign, void* dx) {
  GH_ENTER("ginn_hip_pick_bwd", ctx);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_pick_bwd: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(idx && dout && dx, "ginn_hip_pick_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(cols, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (pick_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               rows, cols, idx, static_cast<const T::storage*>(dout), sign,
                               static_cast<T::storage*>(dx))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick_nlsig_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* x, const int* idx,
                            void* sigm, void* out) {
  GH_ENTER("ginn_hip_pick_nlsig_fwd", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(x && idx && sigm && out, "ginn_hip_pick_nlsig_fwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (pick_nlsig_fwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               n, static_cast<const T::storage*>(x), idx, static_cast<T::storage*>(sigm),
                               static_cast<T::storage*>(out))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_pick_nlsig_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* sigm, const int* idx,
                            const void* dout, void* dx) {
  GH_ENTER("ginn_hip_pick_nlsig_bwd", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(sigm && idx && dout && dx, "ginn_hip_pick_nlsig_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (pick_nlsig_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               n, static_cast<const T::storage*>(sigm), idx, static_cast<const T::storage*>(dout),
                               static_cast<T::storage*>(dx))));
  GH_HIP(hipGetLastError());
  return kOk;
}

static int make_axis_desc(const char* who, int rank, const long long* host_dims, const int* host_summed,
                          AxisDesc* d) {
  GH_CHECK_ARG(rank >= 1 && rank <= 8, "%s: rank %d is not in 1..8", who, rank);
  GH_CHECK_ARG(host_dims && host_summed, "%s: NULL table", who);
  d->rank = rank;
  d->n_in = 1;
  d->n_out = 1;
  for (int a = 0; a < rank; ++a) {
    GH_CHECK_ARG(host_dims[a] >= 0, "%s: negative extent", who);
    d->dim[a] = host_dims[a];
    d->n_in *= host_dims[a];
    if (host_summed[a]) {
      d->out_stride[a] = 0;
    } else {
      d->out_stride[a] = d->n_out;
      d->n_out *= host_dims[a];
    }
  }
  for (int a = rank; a < 8; ++a) {
    d->dim[a] = 1;
    d->out_stride[a] = 0;
  }
  return kOk;
}

int ginn_hip_axis_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank, const long long* host_dims,
                      const int* host_summed, const void* x, void* dst) {
  GH_ENTER("ginn_hip_axis_sum", ctx);
  AxisDesc d;
  if (int rc = make_axis_desc("ginn_hip_axis_sum", rank, host_dims, host_summed, &d)) return rc;
  if (d.n_in == 0 || d.n_out == 0) return kOk;
  GH_CHECK_ARG(x && dst, "ginn_hip_axis_sum: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(d.n_out), kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (axis_sum_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               d, static_cast<const T::storage*>(x), static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_axis_sum_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank, const long long* host_dims,
                          const int* host_summed, const void* dy, void* dx) {
  GH_ENTER("ginn_hip_axis_sum_bwd", ctx);
  AxisDesc d;
  if (int rc = make_axis_desc("ginn_hip_axis_sum_bwd", rank, host_dims, host_summed, &d)) return rc;
  if (d.n_in == 0) return kOk;
  GH_CHECK_ARG(dy && dx, "ginn_hip_axis_sum_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(d.n_in), kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (axis_sum_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               d, static_cast<const T::storage*>(dy), static_cast<T::storage*>(dx))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_variance_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* x, void* mean_out,
                          void* var_out) {
  GH_ENTER("ginn_hip_variance_fwd", ctx);
  GH_CHECK_ARG(n > 0, "ginn_hip_variance_fwd: the variance of nothing");
  GH_CHECK_ARG(x && mean_out && var_out, "ginn_hip_variance_fwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  GH_DISPATCH_DTYPE(dtype, (variance_fwd_kernel<T><<<1, kBlock, 0, ctx->stream>>>(
                               n, static_cast<const T::storage*>(x), static_cast<T::storage*>(mean_out),
                               static_cast<T::storage*>(var_out))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_variance_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, const void* x, const void* mean,
                          const void* dvar, void* dx) {
  GH_ENTER("ginn_hip_variance_bwd", ctx);
  if (n == 0) return kOk;
  GH_CHECK_ARG(x && mean && dvar && dx, "ginn_hip_variance_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (variance_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               n, static_cast<const T::storage*>(x), static_cast<const T::storage*>(mean),
                               static_cast<const T::storage*>(dvar), static_cast<T::storage*>(dx))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_stack(ginn_hip_ctx* ctx, int elem_bytes, size_t sz, size_t count, const void* const* dev_srcs,
                   void* dst) {
  GH_CHECK_ARG(ctx, "ginn_hip_stack: ctx is NULL");
  GH_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, "ginn_hip_stack: element size %d", elem_bytes);
  if (sz == 0 || count == 0) return kOk;
  GH_CHECK_ARG(dev_srcs && dst, "ginn_hip_stack: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(sz * count, kBlock, ctx->num_cus);
  if (elem_bytes == 4)
    stack_kernel<uint32_t><<<grid, kBlock, 0, ctx->stream>>>(sz, count, reinterpret_cast<const uint32_t* const*>(dev_srcs),
                                                            static_cast<uint32_t*>(dst));
  else if (elem_bytes == 2)
    stack_kernel<uint16_t><<<grid, kBlock, 0, ctx->stream>>>(sz, count, reinterpret_cast<const uint16_t* const*>(dev_srcs),
                                                            static_cast<uint16_t*>(dst));
  else
    stack_kernel<uint8_t><<<grid, kBlock, 0, ctx->stream>>>(sz, count, reinterpret_cast<const uint8_t* const*>(dev_srcs),
                                                           static_cast<uint8_t*>(dst));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_stack_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t sz, size_t count, void* const* dev_dsts,
                       const void* src) {
  GH_ENTER("ginn_hip_stack_bwd", ctx);
  if (sz == 0 || count == 0) return kOk;
  GH_CHECK_ARG(dev_dsts && src, "ginn_hip_stack_bwd: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(sz * count, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (stack_bwd_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               sz, count, reinterpret_cast<T::storage* const*>(dev_dsts),
                               static_cast<const T::storage*>(src))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_argmax(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t inner, size_t len, size_t outer, const void* x,
                    long long* out) {
  GH_ENTER("ginn_hip_argmax", ctx);
  GH_CHECK_ARG(len > 0, "ginn_hip_argmax: empty axis");
  if (inner == 0 || outer == 0) return kOk;
  GH_CHECK_ARG(x && out, "ginn_hip_argmax: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(inner * outer, kBlock, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (argmax_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               inner, len, outer, static_cast<const T::storage*>(x), out)));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_row_broadcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, void* dst) {
  GH_ENTER("ginn_hip_row_broadcast", ctx);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_row_broadcast: negative dimension");
  if (rows == 0 || cols == 0) return kOk;
  GH_CHECK_ARG(x && dst, "ginn_hip_row_broadcast: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const size_t n = static_cast<size_t>(rows) * cols;
  GH_DISPATCH_DTYPE(dtype, (row_broadcast_kernel<T><<<grid_for(n, kBlock, ctx->num_cus), kBlock, 0, ctx->stream>>>(
                               rows, n, static_cast<const T::storage*>(x), static_cast<T::storage*>(dst))));
  GH_HIP(hipGetLastError());
  return kOk;
}

int ginn_hip_col_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols, const void* x, void* dst,
                     int accumulate) {
  GH_ENTER("ginn_hip_col_sum", ctx);
  GH_CHECK_ARG(rows >= 0 && cols >= 0, "ginn_hip_col_sum: negative dimension");
  if (cols == 0) return kOk;
  GH_CHECK_ARG(dst && (rows == 0 || x), "ginn_hip_col_sum: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(static_cast<size_t>(cols), kBlock / 64, ctx->num_cus);
  GH_DISPATCH_DTYPE(dtype, (col_sum_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(
                               rows, cols, static_cast<const T::storage*>(x), static_cast<T::storage*>(dst),
                               accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

}  // extern "C"
