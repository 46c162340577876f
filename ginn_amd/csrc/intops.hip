// Arithmetic on ginn::Int (32-bit integer) tensors: the forward passes of Add,
// Subtract, AddScalar / SubtractScalar / ProdScalar, CwiseProd, CwiseProdAdd and
// CwiseMax, which the reference instantiates for Int (test/nodes.cu.cpp:443-640,
// ginn-py/node/common-py.cu.cpp:34-70), and of Select, Mask and UpperTri
// (test/nodes.cu.cpp:825-905, 1555-1580).  Exact integer arithmetic (wrapping on
// overflow, like the reference's int on the device); no gradients exist for Int.
// Index-sized tensors: one element per lane, nothing tuned.
#include "kernel_util.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

template <int OP>
__global__ __launch_bounds__(kBlock) void int_arith_kernel(size_t n, size_t rows, const int* __restrict__ a,
                                                           const int* __restrict__ b, const int* __restrict__ c,
                                                           int ia, int ib, int* __restrict__ dst, int accumulate) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride) {
    int v;
    if (OP == kIntAdd) v = a[i] + (b ? b[i] : 0);
    else if (OP == kIntSub) v = a[i] - b[i];
    else if (OP == kIntMul) v = a[i] * b[i];
    else if (OP == kIntMax) v = max(a[i], b[i]);
    else if (OP == kIntScaleShift) v = ia * a[i] + ib;
    else {  // kIntMulAdd: a (*) (b + ia) + c, b and c per row when rows != 0
      const size_t j = rows ? i % rows : i;
      v = a[i] * (b[j] + ia) + c[j];
    }
    dst[i] = accumulate ? dst[i] + v : v;
  }
}

// dst[i] = cond[i] ? a : b, a branch flagged scalar being one value for every i.
__global__ __launch_bounds__(kBlock) void int_select_kernel(size_t n, const uint8_t* __restrict__ cond,
                                                            const int* a, int a_scalar, const int* b, int b_scalar,
                                                            int* dst) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
    dst[i] = cond[i] ? a[a_scalar ? 0 : i] : b[b_scalar ? 0 : i];
}

// dst[i] = mask[i % mask_size] != 0 ? x[i] : value.
__global__ __launch_bounds__(kBlock) void int_mask_kernel(size_t mask_size, size_t n, const int* __restrict__ mask,
                                                          int value, const int* x, int* dst) {
  const size_t stride = static_cast<size_t>(gridDim.x) * kBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < n; i += stride)
    dst[i] = mask[i % mask_size] != 0 ? x[i] : value;
}

// Column-major n x n: 1 on and above the diagonal, 0 below.
__global__ __launch_bounds__(kBlock) void int_upper_tri_kernel(size_t n, int* dst) {
  const size_t total = n * n, stride = static_cast<size_t>(gridDim.x) * kBlock;
  for (size_t i = static_cast<size_t>(blockIdx.x) * kBlock + threadIdx.x; i < total; i += stride)
    dst[i] = i % n <= i / n ? 1 : 0;
}

}  // namespace

int launch_int_select(ginn_hip_ctx* ctx, size_t n, const unsigned char* cond, const void* a, int a_is_scalar,
                      const void* b, int b_is_scalar, void* dst) {
  GH_HIP(hipSetDevice(ctx->device));
  int_select_kernel<<<grid_for(n, kBlock, ctx->num_cus), kBlock, 0, ctx->stream>>>(
      n, cond, static_cast<const int*>(a), a_is_scalar, static_cast<const int*>(b), b_is_scalar,
      static_cast<int*>(dst));
  GH_HIP(hipGetLastError());
  return kOk;
}

int launch_int_mask(ginn_hip_ctx* ctx, size_t mask_size, size_t n, const void* mask, int value, const void* x,
                    void* dst) {
  GH_HIP(hipSetDevice(ctx->device));
  int_mask_kernel<<<grid_for(n, kBlock, ctx->num_cus), kBlock, 0, ctx->stream>>>(
      mask_size, n, static_cast<const int*>(mask), value, static_cast<const int*>(x), static_cast<int*>(dst));
  GH_HIP(hipGetLastError());
  return kOk;
}

int launch_int_upper_tri(ginn_hip_ctx* ctx, size_t n, void* dst) {
  GH_HIP(hipSetDevice(ctx->device));
  int_upper_tri_kernel<<<grid_for(n * n, kBlock, ctx->num_cus), kBlock, 0, ctx->stream>>>(n, static_cast<int*>(dst));
  GH_HIP(hipGetLastError());
  return kOk;
}

int launch_int_arith(ginn_hip_ctx* ctx, int op, size_t n, size_t rows, const void* a, const void* b, const void* c,
                     int ia, int ib, void* dst, int accumulate) {
  if (n == 0) return kOk;
  if (!a || !dst || ((op == kIntSub || op == kIntMul || op == kIntMax || op == kIntMulAdd) && !b) ||
      (op == kIntMulAdd && !c))
    return fail(kInvalidArgument, "integer arithmetic: NULL operand");
  GH_HIP(hipSetDevice(ctx->device));
  const unsigned grid = grid_for(n, kBlock, ctx->num_cus);
#define GH_INT(OPC)                                                                                               \
  int_arith_kernel<OPC><<<grid, kBlock, 0, ctx->stream>>>(n, rows, static_cast<const int*>(a),                    \
                                                          static_cast<const int*>(b), static_cast<const int*>(c), \
                                                          ia, ib, static_cast<int*>(dst), accumulate)
  switch (op) {
    case kIntAdd: GH_INT(kIntAdd); break;
    case kIntSub: GH_INT(kIntSub); break;
    case kIntMul: GH_INT(kIntMul); break;
    case kIntMax: GH_INT(kIntMax); break;
    case kIntScaleShift: GH_INT(kIntScaleShift); break;
    case kIntMulAdd: GH_INT(kIntMulAdd); break;
    default: return fail(kInvalidArgument, "integer arithmetic: unknown operation %d", op);
  }
#undef GH_INT
  GH_HIP(hipGetLastError());
  return kOk;
}

}  // namespace ginn_hip
