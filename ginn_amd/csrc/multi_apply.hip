// One launch for many independent elementwise operations: the graph executor
// of the host layer collects the element-wise nodes of one height (the gates
// of all sequences of a recurrent step, say) and hands them over as a table.
// Each operation is small (hundreds of elements); what is saved is the launch
// per node.  Two forms: operations of one kind and length over tables of
// pointers (multi_apply), and operations of any kind, length and scalar type,
// one record each (multi_mixed).
#include <algorithm>

#include "common.h"
#include "kernel_util.h"
#include "reduce_rows.h"
#include "vec_access.h"

namespace ginn_hip {
namespace {

constexpr int kBlock = 256;

struct MultiParams {
  void* const* dst;
  const void* const* src0;
  const void* const* src1;
  const void* const* src2;
  size_t n;
  int kind, act, accumulate;
  float value;
};

// What an operation does, apart from where its operands are.
struct OpKind {
  int kind, act, accumulate;
  float value;
};

// N elements of one operation: v = f(s0, s1, s2).  One branch on the kind
// (and one on the activation) for all of them.
template <bool FAST, int N>
__device__ __forceinline__ void multi_values(const OpKind& k, const float (&s0)[N], const float (&s1)[N],
                                             const float (&s2)[N], float (&v)[N]) {
  switch (k.kind) {
    case GINN_HIP_MULTI_FILL:
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = k.value;
      break;
    case GINN_HIP_MULTI_SUM:  // absent sources were read as zeros
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = s0[e] + s1[e] + s2[e];
      break;
    case GINN_HIP_MULTI_PROD:
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = s0[e] * s1[e];
      break;
    case GINN_HIP_MULTI_NONLIN_FWD:
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = s0[e];
      act_forward_n<FAST, N>(k.act, v);
      break;
    default:  // GINN_HIP_MULTI_NONLIN_BWD: dy, x, y
#pragma unroll
      for (int e = 0; e < N; ++e) v[e] = s0[e];
      act_backward_n<FAST, N>(k.act, s1, s2, v);
      break;
  }
}

// One operation of n elements, the blocks of gridDim.x striding over it: eight
// elements at a time with 16-byte accesses when its pointers and length allow
// (large operations then run at memory speed), else one by one.
template <typename T>
__device__ __forceinline__ void apply_one(const OpKind& k, size_t n, void* dst_, const void* s0_, const void* s1_,
                                          const void* s2_, size_t first, size_t step) {
  using S = typename T::storage;
  constexpr bool FAST = kFastMath<T>;
  S* dst = static_cast<S*>(dst_);
  const S* s0 = static_cast<const S*>(s0_);
  const S* s1 = static_cast<const S*>(s1_);
  const S* s2 = static_cast<const S*>(s2_);
  const bool has1 = s1 != nullptr, has2 = s2 != nullptr;
  const uintptr_t bits = reinterpret_cast<uintptr_t>(dst) | reinterpret_cast<uintptr_t>(s0) |
                         reinterpret_cast<uintptr_t>(s1) | reinterpret_cast<uintptr_t>(s2);
  if constexpr (sizeof(S) == 4) {
    // fp32, a short operation (one pass of the lanes covers it): four elements per lane instead of eight.
    // What such an operation costs is the length of the dependent instruction stream of one wave, and the
    // transcendental functions of fp32 are long: with four elements the wave issues half as many
    // instructions, still with four independent chains to fill the pipeline (one element per lane was
    // measured too: no better), and the access is one 16-byte vector per operand either way.
    if (bits % 16 == 0 && n % 4 == 0 && n <= 4 * step) {
      const size_t i = first * 4;
      if (i < n) {
        float a[4], b[4], c[4], d[4], v[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) a[e] = b[e] = c[e] = d[e] = 0.f;
        if (s0) ld<T, 4>(s0 + i, a);
        if (has1) ld<T, 4>(s1 + i, b);
        if (has2) ld<T, 4>(s2 + i, c);
        if (k.accumulate) ld<T, 4>(dst + i, d);
        multi_values<FAST, 4>(k, a, b, c, v);
#pragma unroll
        for (int e = 0; e < 4; ++e) v[e] += d[e];
        st<T, 4>(dst + i, v);
      }
      return;
    }
  }
  if (bits % 16 == 0 && n % 8 == 0) {
    for (size_t i = first * 8; i < n; i += step * 8) {
      float a[8], b[8], c[8], d[8], v[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = b[e] = c[e] = d[e] = 0.f;
      if (s0) ld<T, 8>(s0 + i, a);
      if (has1) ld<T, 8>(s1 + i, b);
      if (has2) ld<T, 8>(s2 + i, c);
      if (k.accumulate) ld<T, 8>(dst + i, d);
      multi_values<FAST, 8>(k, a, b, c, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) v[e] += d[e];
      st<T, 8>(dst + i, v);
    }
    return;
  }
  for (size_t i = first; i < n; i += step) {
    const float a[1] = {s0 ? to_float<T>(s0[i]) : 0.f};
    const float b[1] = {has1 ? to_float<T>(s1[i]) : 0.f};
    const float c[1] = {has2 ? to_float<T>(s2[i]) : 0.f};
    float v[1];
    multi_values<FAST, 1>(k, a, b, c, v);
    if (k.accumulate) v[0] += to_float<T>(dst[i]);
    dst[i] = from_float<T>(v[0]);
  }
}

// Operations of one kind and length: blockIdx.y selects the operation.
template <typename T>
__global__ __launch_bounds__(kBlock) void multi_apply_kernel(MultiParams p) {
  const unsigned op = blockIdx.y;
  const OpKind k{p.kind, p.act, p.accumulate, p.value};
  apply_one<T>(k, p.n, p.dst[op], p.src0 ? p.src0[op] : nullptr, p.src1 ? p.src1[op] : nullptr,
               p.src2 ? p.src2[op] : nullptr, blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x,
               static_cast<size_t>(gridDim.x) * kBlock);
}

// One record with the threads first, first + step, ... striding over it.
// By value: the caller reads a record from LDS in one go, not field by field.
__device__ __forceinline__ void apply_record(const ginn_hip_multi_op op, size_t first, size_t step) {
  const OpKind k{op.kind, op.act, op.accumulate, op.value};
  switch (op.dtype) {
    case GINN_HIP_F32: apply_one<F32>(k, op.n, op.dst, op.src[0], op.src[1], op.src[2], first, step); break;
    case GINN_HIP_F16: apply_one<F16>(k, op.n, op.dst, op.src[0], op.src[1], op.src[2], first, step); break;
    default: apply_one<BF16>(k, op.n, op.dst, op.src[0], op.src[1], op.src[2], first, step); break;
  }
}

// Operations of any kind, length and scalar type, each described by its own
// record: blockIdx.y selects the operation; the grid is sized for the longest
// one, and blocks beyond the length of theirs find nothing to do.
__global__ __launch_bounds__(kBlock) void multi_mixed_kernel(const ginn_hip_multi_op* __restrict__ ops) {
  apply_record(ops[blockIdx.y], blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x,
               static_cast<size_t>(gridDim.x) * kBlock);
}

// Chains of dependent operations: block b runs the records
// [chains[b].first, + count) stage by stage (`reserved` is a record's stage);
// records of one stage are independent of each other, and before the first
// record of a later stage the block waits until the earlier ones are done and
// their stores are visible to all of its waves.  Chains are independent of
// each other, so one launch does the work of as many launches as there are
// stages.  What a stage costs is the latency of its loads, so the records are
// fetched into LDS once, and a stage of several short operations is dealt out
// over the four waves (one operation per wave at a time) instead of running
// them one after the other on the whole block.
constexpr unsigned kChainLds = 64;      // records kept in LDS per batch: one bit each in a 64-bit mask
constexpr size_t kChainWaveOp = 4096;   // longest operation that one wave takes alone

__global__ __launch_bounds__(kBlock) void multi_chain_kernel(const ginn_hip_multi_op* __restrict__ ops,
                                                             const ginn_hip_chain_range* __restrict__ chains) {
  __shared__ ginn_hip_multi_op recs[kChainLds];
  const ginn_hip_chain_range c = chains[blockIdx.x];
  const unsigned wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  constexpr unsigned kWords = sizeof(ginn_hip_multi_op) / 16;  // 16-byte pieces of a record
  for (unsigned base = 0; base < c.count;) {
    // Fetch the next records; a batch ends at a stage boundary unless one
    // stage alone is longer than the buffer.
    const unsigned avail = min(c.count - base, kChainLds);
    __syncthreads();  // the previous batch is done: its stores count as an earlier stage
    const uint4* src = reinterpret_cast<const uint4*>(ops + c.first + base);
    uint4* dst = reinterpret_cast<uint4*>(recs);
    for (unsigned i = threadIdx.x; i < avail * kWords; i += kBlock) dst[i] = src[i];
    __syncthreads();
    // Where the stages begin and which records are long, one bit per record, found by every wave
    // for itself (two LDS reads): the stage loop below then reads nothing.  (Scanning the records
    // for the end of each stage cost more than the stages' arithmetic.)
    const bool present = lane < avail;
    const bool begin = present && (lane == 0 || recs[lane].reserved != recs[lane - 1].reserved);
    const unsigned long long begins = __ballot(begin);
    const unsigned long long longs = __ballot(present && recs[lane].n > kChainWaveOp);
    unsigned take = avail;
    if (base + avail < c.count) {
      const unsigned cut = 63u - static_cast<unsigned>(__builtin_clzll(begins));  // bit 0 is set
      if (cut > 0) take = cut;  // leave the unfinished stage to the next batch
    }
    unsigned i = 0;
    while (i < take) {
      const unsigned long long later = i + 1 < 64 ? begins >> (i + 1) : 0ull;
      unsigned j = later ? i + 1 + static_cast<unsigned>(__builtin_ctzll(later)) : take;
      if (j > take) j = take;
      const unsigned long long stage = (j - i < 64 ? (1ull << (j - i)) - 1 : ~0ull) << i;
      if (j - i >= 2 && !(longs & stage)) {
        for (unsigned r = i + wave; r < j; r += kBlock / 64) apply_record(recs[r], lane, 64);
      } else {
        for (unsigned r = i; r < j; ++r) apply_record(recs[r], threadIdx.x, kBlock);
      }
      i = j;
      // A stage that was cut by the buffer continues in the next batch, which
      // starts with a barrier of its own.
      if (i < take) __syncthreads();
    }
    base += take;
  }
}

// Zero-fills region op = blockIdx.y (bytes[op] bytes at ptrs[op]); blockIdx.x
// strides over it with 16-byte stores where the region allows, bytes otherwise.
__global__ __launch_bounds__(kBlock) void multi_zero_kernel(void* const* __restrict__ ptrs,
                                                            const size_t* __restrict__ bytes) {
  const unsigned op = blockIdx.y;
  char* p = static_cast<char*>(ptrs[op]);
  const size_t n = bytes[op];
  const size_t first = blockIdx.x * static_cast<size_t>(kBlock) + threadIdx.x;
  const size_t step = static_cast<size_t>(gridDim.x) * kBlock;
  if (reinterpret_cast<uintptr_t>(p) % 16 == 0) {
    const size_t vecs = n / 16;
    const uint4 zero = make_uint4(0u, 0u, 0u, 0u);
    for (size_t i = first; i < vecs; i += step) reinterpret_cast<uint4*>(p)[i] = zero;
    for (size_t i = vecs * 16 + first; i < n; i += step) p[i] = 0;
  } else {
    for (size_t i = first; i < n; i += step) p[i] = 0;
  }
}

// dst[r] (+)= sum over k of srcs[k][r]: the row sums of a matrix whose columns
// are scattered in memory (all users of one node adding into its gradient).
// Same geometry as the other row reductions: 64 rows x a chunk of sources per
// block, fp32 partials per chunk, folded by rowred::fold_rows_kernel.
template <typename T>
__global__ __launch_bounds__(rowred::kBlock) void multi_reduce_partial_kernel(int n, int count, int per_chunk,
                                                                              const void* const* __restrict__ srcs,
                                                                              float* __restrict__ partial) {
  using S = typename T::storage;
  __shared__ float red[rowred::kSlices][rowred::kRowsPerBlock];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int r = blockIdx.x * rowred::kRowsPerBlock + tx;
  const int c0 = blockIdx.y * per_chunk;
  const int c1 = min(count, c0 + per_chunk);
  float s = 0.f;
  if (r < n)
#pragma unroll 4
    for (int c = c0 + ty; c < c1; c += rowred::kSlices) s += to_float<T>(static_cast<const S*>(srcs[c])[r]);
  s = rowred::combine(s, red);
  if (ty == 0 && r < n) partial[static_cast<size_t>(blockIdx.y) * n + r] = s;
}

// The same sum in one launch for a small table: a block owns 64 rows, its 16
// waves take every 16th source and combine through LDS (always in the same
// order).  For a few hundred short sources the second launch of the chunked
// form costs more than it saves.
constexpr int kDirectBlock = 1024;
constexpr int kDirectSlices = kDirectBlock / rowred::kRowsPerBlock;
template <typename T>
__global__ __launch_bounds__(kDirectBlock) void multi_reduce_direct_kernel(int n, int count,
                                                                           const void* const* __restrict__ srcs,
                                                                           typename T::storage* dst, int accumulate) {
  using S = typename T::storage;
  __shared__ float red[kDirectSlices][rowred::kRowsPerBlock];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int r = blockIdx.x * rowred::kRowsPerBlock + tx;
  float s = 0.f;
  if (r < n)
#pragma unroll 4
    for (int c = ty; c < count; c += kDirectSlices) s += to_float<T>(static_cast<const S*>(srcs[c])[r]);
  red[ty][tx] = s;
  __syncthreads();
  if (ty == 0 && r < n) {
    float total = 0.f;
#pragma unroll
    for (int k = 0; k < kDirectSlices; ++k) total += red[k][tx];
    if (accumulate) total += to_float<T>(dst[r]);
    dst[r] = from_float<T>(total);
  }
}

}  // namespace
}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" int ginn_hip_multi_reduce(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, int count,
                                     const void* const* dev_srcs, void* dst, int accumulate) {
  GH_CHECK_ARG(ctx, "ginn_hip_multi_reduce: ctx is NULL");
  GH_CHECK_ARG(count >= 0, "ginn_hip_multi_reduce: negative count");
  GH_CHECK_ARG(n <= 0x7fffffff, "ginn_hip_multi_reduce: n does not fit 31 bits");
  if (n == 0) return kOk;
  GH_CHECK_ARG(dst && (count == 0 || dev_srcs), "ginn_hip_multi_reduce: NULL pointer");
  GH_HIP(hipSetDevice(ctx->device));
  const int rows = static_cast<int>(n);
  if (count <= 1024 && static_cast<long long>(rows) * count <= (1ll << 20)) {
    const unsigned blocks = static_cast<unsigned>((rows + rowred::kRowsPerBlock - 1) / rowred::kRowsPerBlock);
    GH_DISPATCH_DTYPE(dtype, (multi_reduce_direct_kernel<T><<<blocks, kDirectBlock, 0, ctx->stream>>>(
                                 rows, count, dev_srcs, static_cast<T::storage*>(dst), accumulate)));
    GH_HIP(hipGetLastError());
    return kOk;
  }
  std::lock_guard<std::mutex> lock(ctx->mutex);  // the workspace holds the partials
  const rowred::Plan plan = rowred::plan(rows, count, ctx->num_cus, ctx->workspace_bytes, 1);
  GH_CHECK_ARG(plan.chunks >= 1, "ginn_hip_multi_reduce: workspace too small for n=%zu", n);
  float* partial = static_cast<float*>(ctx->workspace);
  GH_DISPATCH_DTYPE(dtype, (multi_reduce_partial_kernel<T><<<dim3(plan.row_blocks, plan.chunks), rowred::kBlock, 0,
                                                             ctx->stream>>>(rows, count, plan.cols_per_chunk,
                                                                            dev_srcs, partial)));
  GH_HIP(hipGetLastError());
  GH_DISPATCH_DTYPE(dtype, (rowred::fold_rows_kernel<T><<<plan.fold_blocks, rowred::kFoldBlock, 0, ctx->stream>>>(
      rows, plan.chunks, partial, nullptr, static_cast<T::storage*>(dst), nullptr, accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}


extern "C" int ginn_hip_multi_zero(ginn_hip_ctx* ctx, int count, void* const* dev_ptrs, const size_t* dev_bytes,
                                   size_t max_bytes) {
  GH_CHECK_ARG(ctx, "ginn_hip_multi_zero: ctx is NULL");
  GH_CHECK_ARG(count >= 0, "ginn_hip_multi_zero: negative count");
  if (count == 0 || max_bytes == 0) return kOk;
  GH_CHECK_ARG(count <= 65535, "ginn_hip_multi_zero: at most 65535 regions per launch, got %d", count);
  GH_CHECK_ARG(dev_ptrs && dev_bytes, "ginn_hip_multi_zero: NULL table");
  GH_HIP(hipSetDevice(ctx->device));
  // Blocks for the largest region (16 bytes per thread and step), a few
  // thousand in total at most: the others find nothing beyond their size.
  size_t bx = (max_bytes / 16 + kBlock - 1) / kBlock;
  const size_t cap = std::max<size_t>(1, static_cast<size_t>(ctx->num_cus) * 16 / static_cast<size_t>(count));
  if (bx > cap) bx = cap;
  if (bx < 1) bx = 1;
  multi_zero_kernel<<<dim3(static_cast<unsigned>(bx), static_cast<unsigned>(count)), kBlock, 0, ctx->stream>>>(
      dev_ptrs, dev_bytes);
  GH_HIP(hipGetLastError());
  return kOk;
}

extern "C" int ginn_hip_multi_apply(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, ginn_hip_multi_kind kind,
                                    ginn_hip_act act, int accumulate, float value, size_t n, int count,
                                    void* const* dev_dst, const void* const* dev_src0,
                                    const void* const* dev_src1, const void* const* dev_src2) {
  GH_CHECK_ARG(ctx, "ginn_hip_multi_apply: ctx is NULL");
  GH_CHECK_ARG(count >= 0, "ginn_hip_multi_apply: negative count");
  GH_CHECK_ARG(kind >= GINN_HIP_MULTI_FILL && kind <= GINN_HIP_MULTI_NONLIN_BWD,
               "ginn_hip_multi_apply: unknown kind %d", kind);
  if (n == 0 || count == 0) return kOk;
  GH_CHECK_ARG(count <= 65535, "ginn_hip_multi_apply: at most 65535 operations per launch, got %d", count);
  GH_CHECK_ARG(dev_dst, "ginn_hip_multi_apply: dst table is NULL");
  const bool nonlin = kind == GINN_HIP_MULTI_NONLIN_FWD || kind == GINN_HIP_MULTI_NONLIN_BWD;
  GH_CHECK_ARG(!nonlin || (act >= GINN_HIP_ACT_IDENTITY && act <= GINN_HIP_ACT_SQRT && act != GINN_HIP_ACT_SOFTMAX),
               "ginn_hip_multi_apply: activation %d is not elementwise", act);
  GH_CHECK_ARG(kind == GINN_HIP_MULTI_FILL || dev_src0, "ginn_hip_multi_apply: src0 table is NULL");
  GH_CHECK_ARG(kind != GINN_HIP_MULTI_PROD || dev_src1, "ginn_hip_multi_apply: a product needs src1");
  if (kind == GINN_HIP_MULTI_NONLIN_BWD) {
    const bool needs_x = act_backward_requires_input(act);
    const bool needs_y = act == GINN_HIP_ACT_TANH || act == GINN_HIP_ACT_RELU || act == GINN_HIP_ACT_SIGMOID ||
                         act == GINN_HIP_ACT_SQRT;
    GH_CHECK_ARG(!needs_x || dev_src1, "ginn_hip_multi_apply: this activation's backward needs x (src1)");
    GH_CHECK_ARG(!needs_y || dev_src2, "ginn_hip_multi_apply: this activation's backward needs y (src2)");
  }
  GH_HIP(hipSetDevice(ctx->device));
  MultiParams p;
  p.dst = dev_dst;
  p.src0 = dev_src0;
  p.src1 = dev_src1;
  p.src2 = dev_src2;
  p.n = n;
  p.kind = kind;
  p.act = act;
  p.accumulate = accumulate;
  p.value = value;
  // Blocks for 8 elements per thread and step, about 16 blocks per CU over
  // all operations: small operations get one block, large ones stride.
  size_t bx = (n + 8 * kBlock - 1) / (8 * kBlock);
  const size_t cap = std::max<size_t>(1, static_cast<size_t>(ctx->num_cus) * 16 / static_cast<size_t>(count));
  if (bx > cap) bx = cap;
  const dim3 grid(static_cast<unsigned>(bx), static_cast<unsigned>(count));
  GH_DISPATCH_DTYPE(dtype, (multi_apply_kernel<T><<<grid, kBlock, 0, ctx->stream>>>(p)));
  GH_HIP(hipGetLastError());
  return kOk;
}

extern "C" int ginn_hip_multi_mixed(ginn_hip_ctx* ctx, int count, const ginn_hip_multi_op* dev_ops, size_t max_n) {
  GH_CHECK_ARG(ctx, "ginn_hip_multi_mixed: ctx is NULL");
  GH_CHECK_ARG(count >= 0, "ginn_hip_multi_mixed: negative count");
  if (count == 0 || max_n == 0) return kOk;
  GH_CHECK_ARG(count <= 65535, "ginn_hip_multi_mixed: at most 65535 operations per launch, got %d", count);
  GH_CHECK_ARG(dev_ops, "ginn_hip_multi_mixed: table is NULL");
  GH_HIP(hipSetDevice(ctx->device));
  // As multi_apply, sized for the longest operation.
  size_t bx = (max_n + 8 * kBlock - 1) / (8 * kBlock);
  const size_t cap = std::max<size_t>(1, static_cast<size_t>(ctx->num_cus) * 16 / static_cast<size_t>(count));
  if (bx > cap) bx = cap;
  multi_mixed_kernel<<<dim3(static_cast<unsigned>(bx), static_cast<unsigned>(count)), kBlock, 0, ctx->stream>>>(
      dev_ops);
  GH_HIP(hipGetLastError());
  return kOk;
}

extern "C" int ginn_hip_multi_chain(ginn_hip_ctx* ctx, int chains, const ginn_hip_chain_range* dev_chains,
                                    const ginn_hip_multi_op* dev_ops) {
  GH_CHECK_ARG(ctx, "ginn_hip_multi_chain: ctx is NULL");
  GH_CHECK_ARG(chains >= 0, "ginn_hip_multi_chain: negative count");
  if (chains == 0) return kOk;
  GH_CHECK_ARG(dev_chains && dev_ops, "ginn_hip_multi_chain: NULL table");
  GH_HIP(hipSetDevice(ctx->device));
  multi_chain_kernel<<<dim3(static_cast<unsigned>(chains)), kBlock, 0, ctx->stream>>>(dev_ops, dev_chains);
  GH_HIP(hipGetLastError());
  return kOk;
}
