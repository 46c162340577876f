// Postponed second halves of row reductions.  A row sum over a column-major
// matrix is two launches: per-chunk partial sums, then a fold of the chunks.
// The fold is a few microseconds of launch and latency for a few kilobytes of
// work; a backward pass makes one per bias gradient (AffineNode::backward_,
// ginn/node/affine.h:117-122) and per LayerNorm scale / shift gradient.  A
// caller that does not need those sums before the end of the pass asks for the
// folds to wait (ginn_hip_defer_folds) and runs them all as one launch
// (ginn_hip_flush_folds).  The sums are the same bits either way.
#include <algorithm>

#include "common.h"
#include "kernel_util.h"
#include "reduce_rows.h"

namespace ginn_hip {
namespace {

constexpr int kMaxJobs = 16;                    // per launch: the jobs travel as kernel arguments
constexpr size_t kArenaBytes = size_t(8) << 20;  // partial sums of the queued jobs

struct FoldJobs {
  ginn_hip_fold_job job[kMaxJobs];
};

__global__ __launch_bounds__(rowred::kFoldBlock) void multi_fold_kernel(FoldJobs jobs) {
  __shared__ float red[2][rowred::kFoldSlices][rowred::kFoldRows];
  const ginn_hip_fold_job& j = jobs.job[blockIdx.y];
  if (static_cast<int>(blockIdx.x) * rowred::kFoldRows >= j.rows) return;  // whole block: no barrier is skipped
  switch (j.dtype) {
    case GINN_HIP_F32:
      rowred::fold_rows_block<F32>(blockIdx.x, j.rows, j.chunks, j.part_a, j.part_b, static_cast<float*>(j.dst_a),
                                   static_cast<float*>(j.dst_b), j.accumulate, red);
      break;
    case GINN_HIP_F16:
      rowred::fold_rows_block<F16>(blockIdx.x, j.rows, j.chunks, j.part_a, j.part_b, static_cast<uint16_t*>(j.dst_a),
                                   static_cast<uint16_t*>(j.dst_b), j.accumulate, red);
      break;
    default:
      rowred::fold_rows_block<BF16>(blockIdx.x, j.rows, j.chunks, j.part_a, j.part_b,
                                    static_cast<uint16_t*>(j.dst_a), static_cast<uint16_t*>(j.dst_b), j.accumulate,
                                    red);
      break;
  }
}

// Depth of ginn_hip_defer_folds(ctx, 1) calls of this host thread: only its own
// calls wait, another thread sharing the context keeps the two-launch form.
thread_local int tl_defer_depth = 0;

}  // namespace

namespace rowred {

int flush_folds(ginn_hip_ctx* ctx) {
  ginn_hip_fold_queue& q = ctx->folds;
  if (q.jobs.empty()) return kOk;
  GH_HIP(hipSetDevice(ctx->device));
  for (size_t first = 0; first < q.jobs.size(); first += kMaxJobs) {
    const size_t count = std::min<size_t>(kMaxJobs, q.jobs.size() - first);
    FoldJobs args;
    int blocks = 1;
    for (size_t i = 0; i < count; ++i) {
      args.job[i] = q.jobs[first + i];
      blocks = std::max(blocks, (args.job[i].rows + kFoldRows - 1) / kFoldRows);
    }
    multi_fold_kernel<<<dim3(blocks, static_cast<unsigned>(count)), kFoldBlock, 0, ctx->stream>>>(args);
    GH_HIP(hipGetLastError());
  }
  q.jobs.clear();
  q.used = 0;
  return kOk;
}

Partials take_partials(ginn_hip_ctx* ctx, size_t bytes) {
  ginn_hip_fold_queue& q = ctx->folds;
  if (tl_defer_depth > 0 && bytes <= kArenaBytes) {
    if (!q.arena) {
      void* p = nullptr;
      if (hipMalloc(&p, kArenaBytes) == hipSuccess) {
        q.arena = static_cast<char*>(p);
        q.arena_bytes = kArenaBytes;
      } else {
        (void)hipGetLastError();  // no room: this reduction folds at once
      }
    }
    const size_t need = (bytes + 255) & ~size_t(255);
    if (q.arena && q.used + need > q.arena_bytes && flush_folds(ctx) != kOk) return {nullptr, false};
    if (q.arena && q.used + need <= q.arena_bytes) {
      float* base = reinterpret_cast<float*>(q.arena + q.used);
      q.used += need;
      return {base, true};
    }
  }
  return {static_cast<float*>(ctx->workspace), false};
}

int finish(ginn_hip_ctx* ctx, const ginn_hip_fold_job& job, bool deferred) {
  if (deferred) {
    // Two jobs of one launch must not add into the same destination.
    ginn_hip_fold_queue& q = ctx->folds;
    for (const ginn_hip_fold_job& other : q.jobs) {
      const void* taken[2] = {other.dst_a, other.dst_b};
      bool clash = false;
      for (const void* t : taken) clash = clash || (t && (t == job.dst_a || t == job.dst_b));
      if (clash) {
        // The queued jobs go first; the new one keeps its partial sums, which
        // lie in front of q.used, so the area is not handed out again before it ran.
        const size_t used = q.used;
        if (int rc = flush_folds(ctx)) return rc;
        q.used = used;
        break;
      }
    }
    q.jobs.push_back(job);
    return kOk;
  }
  const int blocks = (job.rows + kFoldRows - 1) / kFoldRows;
  GH_DISPATCH_DTYPE(job.dtype, (fold_rows_kernel<T><<<blocks, kFoldBlock, 0, ctx->stream>>>(
      job.rows, job.chunks, job.part_a, job.part_b, static_cast<T::storage*>(job.dst_a),
      static_cast<T::storage*>(job.dst_b), job.accumulate)));
  GH_HIP(hipGetLastError());
  return kOk;
}

}  // namespace rowred
}  // namespace ginn_hip

using namespace ginn_hip;

extern "C" {

int ginn_hip_defer_folds(ginn_hip_ctx* ctx, int on) {
  GH_CHECK_ARG(ctx, "ginn_hip_defer_folds: ctx is NULL");
  if (on) {
    ++tl_defer_depth;
  } else {
    GH_CHECK_ARG(tl_defer_depth > 0, "ginn_hip_defer_folds: switched off more often than on");
    --tl_defer_depth;
  }
  return kOk;
}

int ginn_hip_flush_folds(ginn_hip_ctx* ctx) {
  GH_CHECK_ARG(ctx, "ginn_hip_flush_folds: ctx is NULL");
  std::lock_guard<std::mutex> lock(ctx->mutex);
  return rowred::flush_folds(ctx);
}

int ginn_hip_pending_folds(ginn_hip_ctx* ctx, int* count) {
  GH_CHECK_ARG(ctx && count, "ginn_hip_pending_folds: NULL argument");
  std::lock_guard<std::mutex> lock(ctx->mutex);
  *count = static_cast<int>(ctx->folds.jobs.size());
  return kOk;
}

}  // extern "C"
