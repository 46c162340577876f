// Host-side selection of the generic product kernel variant.
#include "gemm_generic.h"

namespace ginn_hip {
namespace {

using namespace generic;

template <typename T>
int launch_dtype(ginn_hip_ctx* ctx, const GemmArgs& a) {
  constexpr int VEC = Cfg<T>::VEC;
  const size_t es = sizeof(typename T::storage);
  KParams p;
  p.A = a.A;
  p.B = a.B;
  p.C = a.C;
  p.m = a.m;
  p.n = a.n;
  p.k = a.k;
  p.lda = a.lda;
  p.ldb = a.ldb;
  p.ldc = a.ldc;
  p.sa = a.stride_a;
  p.sb = a.stride_b;
  p.sc = a.stride_c;
  p.beta = a.beta;
  p.bias = a.bias;
  p.pre = a.pre;
  p.act = a.act;
  p.bcols = a.bcols;
  p.ccols = a.ccols;
  p.acols = a.acols;

  const bool akc = a.op_a == GINN_HIP_OP_T;  // A stored [k x m]: K contiguous
  const bool bkc = a.op_b == GINN_HIP_OP_N;  // B stored [k x n]: K contiguous
  auto aligned = [&](const void* ptr, int ld, long long stride, int contiguous_extent) {
    return reinterpret_cast<uintptr_t>(ptr) % 16 == 0 && ld % VEC == 0 &&
           contiguous_extent % VEC == 0 && (a.batch <= 1 || stride % VEC == 0);
  };
  const bool b_ok = a.bcols ? (a.cols_vec_ld && (bkc ? a.k : a.n) % VEC == 0)
                             : aligned(a.B, a.ldb, a.stride_b, bkc ? a.k : a.n);
  const bool a_ok = a.acols ? (a.cols_vec_ld && a.m % VEC == 0) : aligned(a.A, a.lda, a.stride_a, akc ? a.k : a.m);
  const bool vec_ld = a_ok && b_ok;
  const uintptr_t c_align = 4 * es;
  if (a.ccols)
    p.vec_c = a.cols_vec_c;
  else
    p.vec_c = reinterpret_cast<uintptr_t>(a.C) % c_align == 0 && a.ldc % 4 == 0 &&
              (a.batch <= 1 || a.stride_c % 4 == 0) &&
              (a.pre == nullptr || reinterpret_cast<uintptr_t>(a.pre) % c_align == 0);

  // 128 x 128 tiles when they fill the machine, 64 x 64 otherwise.
  const long long tiles128 = (long long)((a.m + 127) / 128) * ((a.n + 127) / 128) * a.batch;
  const bool big = a.m > 64 && a.n > 64 && tiles128 >= ctx->num_cus;
  // Too few 64 x 64 tiles for the machine: split K over blockIdx.z, fp32
  // partials in the workspace, folded by a second kernel.
  p.splits = 1;
  p.k_chunk = 0;
  p.partial = nullptr;
  const long long tiles64 = (long long)((a.m + 63) / 64) * ((a.n + 63) / 64);
  std::unique_lock<std::mutex> lock(ctx->mutex, std::defer_lock);
  // A block walks its K range at a few hundred ns per 16 or 32 values whatever
  // the shape, and a fold costs a launch (4-5 us) plus the partials' way
  // through memory.  With tiles for at most a quarter of the CUs the partials
  // are small and the walk is everything: split down to 32 values of K per
  // block.  With more tiles a split has to save 256 values to pay.
  constexpr int BK = Cfg<T>::BK;
  const bool few_tiles = tiles64 * 4 <= ctx->num_cus;
  const int min_chunk = few_tiles ? 32 : 256;
  if (!big && a.batch == 1 && !a.cols_in_workspace && (!a.ccols || a.pre == nullptr) && tiles64 < ctx->num_cus &&
      a.k >= (few_tiles ? 128 : 512)) {
    long long splits = (2ll * ctx->num_cus + tiles64 - 1) / tiles64;
    if (splits > a.k / min_chunk) splits = a.k / min_chunk;
    if (splits > 64) splits = 64;
    const size_t per_split = (size_t)a.m * a.n * sizeof(float);
    if (splits * per_split > ctx->workspace_bytes) splits = ctx->workspace_bytes / per_split;
    // The partial sums go through memory twice (written here, read by the
    // fold): beyond a few MiB that costs more than the shorter walk saves.
    constexpr size_t kPartialBudget = size_t(4) << 20;
    if (few_tiles && splits * per_split > kPartialBudget) splits = kPartialBudget / per_split;
    if (splits > 1) {
      int chunk = (int)((a.k + splits - 1) / splits);
      chunk = (chunk + BK - 1) / BK * BK;
      p.splits = (a.k + chunk - 1) / chunk;
      p.k_chunk = chunk;
      p.partial = static_cast<float*>(ctx->workspace);
      if (p.splits > 1) lock.lock();  // the workspace is shared
      else p.splits = 1;
    }
  }
  if (vec_ld) return launch_variant<T, true>(ctx, p, a.batch, akc, bkc, big);
  return launch_variant<T, false>(ctx, p, a.batch, akc, bkc, big);
}

}  // namespace

int launch_splitk_reduce(ginn_hip_ctx* ctx, const GemmArgs& a, int splits, const float* partial) {
  using namespace generic;
  KParams p{};
  p.C = a.C;
  p.m = a.m;
  p.n = a.n;
  p.ldc = a.ldc;
  p.beta = a.beta;
  p.bias = a.bias;
  p.pre = a.pre;
  p.act = a.act;
  p.splits = splits;
  p.partial = const_cast<float*>(partial);
  switch (a.dtype) {
    case GINN_HIP_F32: return launch_reduce<F32>(ctx, p);
    case GINN_HIP_F16: return launch_reduce<F16>(ctx, p);
    case GINN_HIP_BF16: return launch_reduce<BF16>(ctx, p);
    default: return fail(kInvalidArgument, "split-K reduce: unknown dtype %d", a.dtype);
  }
}

int launch_gemm_generic(ginn_hip_ctx* ctx, const GemmArgs& a) {
  switch (a.dtype) {
    case GINN_HIP_F32:
      return launch_dtype<F32>(ctx, a);
    case GINN_HIP_F16:
      return launch_dtype<F16>(ctx, a);
    case GINN_HIP_BF16:
      return launch_dtype<BF16>(ctx, a);
    default:
      return fail(kInvalidArgument, "gemm: unknown dtype %d", a.dtype);
  }
}

}  // namespace ginn_hip
