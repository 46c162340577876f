// Shared declarations of libginn_hip.so: context, error plumbing, scalar
// helpers and the device-side nonlinearity formulas.
#ifndef GINN_HIP_COMMON_H
#define GINN_HIP_COMMON_H

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <map>
#include <atomic>
#include <mutex>
#include <unordered_map>
#include <vector>

#include "../../include/ginn_hip.h"

namespace ginn_hip {

// ---------------------------------------------------------------------------
// Errors
// ---------------------------------------------------------------------------

enum Status : int {
  kOk = 0,
  kInvalidArgument = 1,
  kHipError = 2,
  kOutOfMemory = 3,
  kUnsupported = 4
};

// Stores a printf-formatted message for ginn_hip_last_error() and returns code.
int fail(int code, const char* fmt, ...);
void clear_error();

#define GH_CHECK_ARG(cond, ...)                                                \
  do {                                                                         \
    if (!(cond)) return ::ginn_hip::fail(::ginn_hip::kInvalidArgument, __VA_ARGS__); \
  } while (0)

#define GH_HIP(stmt)                                                           \
  do {                                                                         \
    hipError_t e__ = (stmt);                                                   \
    if (e__ != hipSuccess)                                                     \
      return ::ginn_hip::fail(::ginn_hip::kHipError, "%s failed: %s (%s:%d)",  \
                              #stmt, hipGetErrorString(e__), __FILE__,         \
                              __LINE__);                                       \
  } while (0)

}  // namespace ginn_hip

// ---------------------------------------------------------------------------
// Context
// ---------------------------------------------------------------------------

// Free device blocks kept for reuse, by block size.  Every block is used on the
// context's one stream only, so a block released by the host may be handed out
// again at once: whatever still reads it was enqueued earlier on that stream.
// Blocks of up to 64 KiB are cut from 2 MiB allocations ("slabs") of their size
// class, next to each other in address order: a graph of a hundred thousand
// small tensors then costs a few hundred driver allocations instead of one per
// tensor, and tensors made one after the other share pages.
struct ginn_hip_slab {
  size_t block = 0;   // size class
  size_t carved = 0;  // bytes handed out so far (blocks are cut front to back)
  size_t live = 0;    // blocks in use; a slab without any can go back to the driver
};
struct ginn_hip_pool {
  std::mutex mutex;
  std::unordered_map<size_t, std::vector<void*>> free_blocks;  // block size -> blocks
  std::unordered_map<void*, size_t> block_size;                // every live or cached block of the pool
  std::map<uintptr_t, ginn_hip_slab> slabs;                    // by base address
  std::unordered_map<size_t, uintptr_t> open_slab;             // size class -> the slab being cut
  size_t cached_bytes = 0;
  size_t limit_bytes = size_t(8) << 30;  // beyond this, released blocks go back to the driver
  bool enabled = true;
};

// Second halves of row reductions that a caller has asked to postpone
// (ginn_hip_defer_folds): each job folds `chunks` fp32 partial rows into up to
// two destinations; ginn_hip_flush_folds runs all of them in one launch.
struct ginn_hip_fold_job {
  int dtype, rows, chunks, accumulate;
  const float* part_a;
  const float* part_b;
  void* dst_a;
  void* dst_b;
};
struct ginn_hip_fold_queue {
  std::vector<ginn_hip_fold_job> jobs;
  char* arena = nullptr;  // partial sums of the queued jobs
  size_t arena_bytes = 0, used = 0;
};

struct ginn_hip_ctx {
  int device = 0;
  hipStream_t stream = nullptr;
  bool owns_stream = false;
  // Device workspace: staging of grouped-GEMM tables and split-K partials.
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  // Pinned host mirror used to upload small tables without a pageable copy.
  void* host_staging = nullptr;
  size_t host_staging_bytes = 0;
  size_t host_staging_used = 0;  // ring cursor
  hipEvent_t staging_event = nullptr;
  hipEvent_t order_event = nullptr;  // ginn_hip_ctx_wait_for with this context as the signaler
  std::mutex mutex;  // serialises workspace users across host threads
  hipEvent_t events[64] = {};
  int num_cus = 256;
  bool may_allocate = true;  // false for the stack context of the entry point that must not allocate
  size_t gemm_temp_budget = size_t(2) << 30;  // ginn_hip_gemm_temp_budget
  ginn_hip_pool pool;
  ginn_hip_fold_queue folds;  // guarded by `mutex`
};

// A recorded sequence of launches on a context's stream.
struct ginn_hip_graph {
  ginn_hip_ctx* ctx = nullptr;
  hipGraph_t graph = nullptr;
  hipGraphExec_t exec = nullptr;
};

struct ginn_hip_arena {
  ginn_hip_ctx* ctx = nullptr;
  char* base = nullptr;
  size_t size = 0;
  size_t used = 0;
  size_t alignment = 1;  // start of every block; 1 = byte-exact bump
};

namespace ginn_hip {

// ---------------------------------------------------------------------------
// Scalars.  16-bit types travel as raw uint16_t; all arithmetic is fp32.
// ---------------------------------------------------------------------------

struct F32 {
  using storage = float;
  static constexpr int kDtype = GINN_HIP_F32;
};
struct F16 {
  using storage = uint16_t;
  static constexpr int kDtype = GINN_HIP_F16;
};
struct BF16 {
  using storage = uint16_t;
  static constexpr int kDtype = GINN_HIP_BF16;
};

// Raises a kernel's limit of dynamic LDS once per device and kernel (`done`
// is that kernel's own mask of devices): the runtime call costs the host most
// of a microsecond, which a product of a few microseconds cannot hide.
inline hipError_t allow_dynamic_lds(std::atomic<unsigned long long>& done, int device, const void* fn, int bytes) {
  const unsigned long long bit = 1ull << (device & 63);
  if (done.load(std::memory_order_acquire) & bit) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e == hipSuccess) done.fetch_or(bit, std::memory_order_release);
  return e;
}

inline size_t dtype_size(int dtype) { return dtype == GINN_HIP_F32 ? 4 : 2; }
inline bool dtype_valid(int dtype) {
  return dtype == GINN_HIP_F32 || dtype == GINN_HIP_F16 ||
         dtype == GINN_HIP_BF16;
}

template <typename T>
__device__ __forceinline__ float to_float(typename T::storage v);
template <>
__device__ __forceinline__ float to_float<F32>(float v) {
  return v;
}
template <>
__device__ __forceinline__ float to_float<F16>(uint16_t v) {
  return static_cast<float>(__builtin_bit_cast(_Float16, v));
}
template <>
__device__ __forceinline__ float to_float<BF16>(uint16_t v) {
  return __builtin_bit_cast(float, static_cast<uint32_t>(v) << 16);
}

template <typename T>
__device__ __forceinline__ typename T::storage from_float(float v);
template <>
__device__ __forceinline__ float from_float<F32>(float v) {
  return v;
}
template <>
__device__ __forceinline__ uint16_t from_float<F16>(float v) {
  return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
}
template <>
__device__ __forceinline__ uint16_t from_float<BF16>(float v) {
  // The hardware conversion of gfx950 (v_cvt_pk_bf16_f32): round to nearest
  // even, NaN stays NaN.
  return __builtin_bit_cast(uint16_t, static_cast<__bf16>(v));
}

// ---------------------------------------------------------------------------
// Nonlinearities (forward on the pre-activation x; backward factor from x, y).
// Formulas follow ginn/nonlin.h:67-300 evaluated in fp32.
//
// FAST selects the transcendental functions: the full routines for fp32
// storage, and for the 16-bit types -- which keep 8 or 11 significant bits of
// the result -- forms built on the hardware's exp2 and reciprocal (absolute
// error about 2e-7), a fifth of the instructions.  An epilogue or an
// element-wise kernel of a 16-bit type handles twice the elements per byte
// and is otherwise bound by these functions instead of by memory.
//
// The `_n` forms take a vector and branch on the activation ONCE: with the
// branch inside the element loop a fused bias + ReLU epilogue cost 40 % more
// than the bias alone.
// ---------------------------------------------------------------------------

template <typename T>
constexpr bool kFastMath = sizeof(typename T::storage) == 2;

template <bool FAST>
__device__ __forceinline__ float exp_as(float x) {
  if constexpr (FAST) return __expf(x);
  else return expf(x);
}

template <bool FAST>
__device__ __forceinline__ float tanh_as(float x) {
  if constexpr (FAST) {
    // 1 - 2 / (1 + e^(2|x|)), and x - x^3 / 3 where that difference would
    // lose the small value.
    const float ax = fabsf(x);
    const float big = 1.f - 2.f * __builtin_amdgcn_rcpf(1.f + __expf(2.f * ax));
    const float small = ax * (1.f - ax * ax * (1.f / 3.f));
    return copysignf(ax < 0.02f ? small : big, x);
  } else {
    return tanhf(x);
  }
}

template <bool FAST>
__device__ __forceinline__ float erf_as(float x) {
  if constexpr (FAST) {
    // Abramowitz & Stegun 7.1.26, |error| <= 1.5e-7.
    const float ax = fabsf(x);
    const float t = __builtin_amdgcn_rcpf(1.f + 0.3275911f * ax);
    const float poly =
        t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
    return copysignf(1.f - poly * __expf(-ax * ax), x);
  } else {
    return erff(x);
  }
}

// One value, activation known at compile time.
template <bool FAST, int ACT>
__device__ __forceinline__ float act_forward_c(float x) {
  if constexpr (ACT == GINN_HIP_ACT_TANH) {
    return tanh_as<FAST>(x);
  } else if constexpr (ACT == GINN_HIP_ACT_RELU) {
    return fmaxf(x, 0.f);
  } else if constexpr (ACT == GINN_HIP_ACT_SIGMOID) {
    // ginn/nonlin.h:141-144: 0.5 * tanh(0.5 x) + 0.5
    return 0.5f * tanh_as<FAST>(0.5f * x) + 0.5f;
  } else if constexpr (ACT == GINN_HIP_ACT_GELU) {
    // ginn/nonlin.h:281-283
    return 0.5f * x * (1.f + erf_as<FAST>(x * 0.70710678118654752440f));
  } else if constexpr (ACT == GINN_HIP_ACT_GELU2) {
    // ginn/nonlin.h:250-254
    const float a = 0.79788456080286535588f;  // sqrt(2/pi)
    const float b = 0.044715f;
    return 0.5f * x * (1.f + tanh_as<FAST>(a * (x + b * x * x * x)));
  } else if constexpr (ACT == GINN_HIP_ACT_LOG) {
    return logf(x);
  } else if constexpr (ACT == GINN_HIP_ACT_SQRT) {
    return sqrtf(x);
  } else {
    return x;
  }
}

// d act(x) / dx expressed with whichever of x (input) and y (output) the
// reference's backward uses (ginn/nonlin.h, the `backward` of each op).
template <bool FAST, int ACT>
__device__ __forceinline__ float act_derivative_c(float x, float y) {
  if constexpr (ACT == GINN_HIP_ACT_TANH) {
    return 1.f - y * y;
  } else if constexpr (ACT == GINN_HIP_ACT_RELU) {
    return y > 0.f ? 1.f : 0.f;
  } else if constexpr (ACT == GINN_HIP_ACT_SIGMOID) {
    return y * (1.f - y);
  } else if constexpr (ACT == GINN_HIP_ACT_GELU) {
    // ginn/nonlin.h:290-296
    const float c = 0.39894228040143267794f;  // 1/sqrt(2 pi)
    if constexpr (FAST) {
      // erf_as(x / sqrt 2) and the density share their exponential, e^(-x^2 / 2): one exp2 and one
      // reciprocal per element (the gradient of a 3072 x 4096 GELU layer is bound by these, not by memory).
      const float e = __expf(-0.5f * x * x);
      const float t = __builtin_amdgcn_rcpf(1.f + (0.3275911f * 0.70710678118654752440f) * fabsf(x));
      const float poly =
          t * (0.254829592f + t * (-0.284496736f + t * (1.421413741f + t * (-1.453152027f + t * 1.061405429f))));
      const float erf = copysignf(1.f - poly * e, x);
      return 0.5f * (1.f + erf) + x * e * c;
    } else {
      return 0.5f * (1.f + erf_as<FAST>(x * 0.70710678118654752440f)) + x * exp_as<FAST>(-0.5f * x * x) * c;
    }
  } else if constexpr (ACT == GINN_HIP_ACT_GELU2) {
    // Same function as ginn/nonlin.h:262-266, written without the division
    // by x: with t = tanh(u), u = a (x + b x^3):
    //   d/dx = 0.5 (1 + t) + 0.5 x (1 - t^2) a (1 + 3 b x^2)
    const float a = 0.79788456080286535588f;
    const float b = 0.044715f;
    const float t = tanh_as<FAST>(a * (x + b * x * x * x));
    return 0.5f * (1.f + t) + 0.5f * x * (1.f - t * t) * a * (1.f + 3.f * b * x * x);
  } else if constexpr (ACT == GINN_HIP_ACT_LOG) {
    return 1.f / x;
  } else if constexpr (ACT == GINN_HIP_ACT_SQRT) {
    return 0.5f / y;
  } else {
    return 1.f;
  }
}

// Runs BODY with the activation as the compile-time constant ACT.
#define GH_SWITCH_ACT(act, ...)                                                      \
  switch (act) {                                                                     \
    case GINN_HIP_ACT_TANH: { constexpr int ACT = GINN_HIP_ACT_TANH; __VA_ARGS__; } break;       \
    case GINN_HIP_ACT_RELU: { constexpr int ACT = GINN_HIP_ACT_RELU; __VA_ARGS__; } break;       \
    case GINN_HIP_ACT_SIGMOID: { constexpr int ACT = GINN_HIP_ACT_SIGMOID; __VA_ARGS__; } break; \
    case GINN_HIP_ACT_GELU: { constexpr int ACT = GINN_HIP_ACT_GELU; __VA_ARGS__; } break;       \
    case GINN_HIP_ACT_GELU2: { constexpr int ACT = GINN_HIP_ACT_GELU2; __VA_ARGS__; } break;     \
    case GINN_HIP_ACT_LOG: { constexpr int ACT = GINN_HIP_ACT_LOG; __VA_ARGS__; } break;         \
    case GINN_HIP_ACT_SQRT: { constexpr int ACT = GINN_HIP_ACT_SQRT; __VA_ARGS__; } break;       \
    default: { constexpr int ACT = GINN_HIP_ACT_IDENTITY; __VA_ARGS__; } break;               \
  }

// v[e] = act(v[e]) for a vector, one branch for all of it.
template <bool FAST, int N>
__device__ __forceinline__ void act_forward_n(int act, float (&v)[N]) {
  GH_SWITCH_ACT(act, {
    _Pragma("unroll") for (int e = 0; e < N; ++e) v[e] = act_forward_c<FAST, ACT>(v[e]);
  })
}

// g[e] *= act'(x[e], y[e]) for a vector, one branch for all of it.
template <bool FAST, int N>
__device__ __forceinline__ void act_backward_n(int act, const float (&x)[N], const float (&y)[N], float (&g)[N]) {
  GH_SWITCH_ACT(act, {
    _Pragma("unroll") for (int e = 0; e < N; ++e) g[e] *= act_derivative_c<FAST, ACT>(x[e], y[e]);
  })
}

// Single values (edge paths, scalar kernels).
template <bool FAST>
__device__ __forceinline__ float act_forward(int act, float x) {
  float v[1] = {x};
  act_forward_n<FAST, 1>(act, v);
  return v[0];
}
template <bool FAST>
__device__ __forceinline__ float act_derivative(int act, float x, float y) {
  const float xs[1] = {x}, ys[1] = {y};
  float g[1] = {1.f};
  act_backward_n<FAST, 1>(act, xs, ys, g);
  return g[0];
}

inline bool act_backward_requires_input(int act) {
  return act == GINN_HIP_ACT_GELU || act == GINN_HIP_ACT_GELU2 ||
         act == GINN_HIP_ACT_SOFTMAX || act == GINN_HIP_ACT_LOG;
}

// ---------------------------------------------------------------------------
// Internal launchers shared between translation units.
// ---------------------------------------------------------------------------

struct GemmArgs {
  int dtype;
  int op_a, op_b;
  int m, n, k;
  const void* A;
  int lda;
  long long stride_a;
  const void* B;
  int ldb;
  long long stride_b;
  float beta;
  void* C;
  int ldc;
  long long stride_c;
  int batch;
  // Two-level batch (batch_inner > 0): slice z of the `batch` slices lies at
  // (z % batch_inner) * stride + (z / batch_inner) * stride2 of each operand.  Only launch_gemm_bsmall
  // reads these; ginn_hip_gemm_strided_batched2 runs everything else level by level.
  int batch_inner = 0;
  long long stride_a2 = 0, stride_b2 = 0, stride_c2 = 0;
  // Optional epilogue: C = act(acc + beta*C + bias[row]); `pre` (same ld and
  // stride as C) receives the value before the activation.
  const void* bias = nullptr;
  void* pre = nullptr;
  int act = GINN_HIP_ACT_IDENTITY;
  // Gathered operands: device tables with the base of every stored column of
  // B (n entries when op_b is N, k entries when it is T) and of every column
  // of the output (n entries).  bcols replaces B/ldb, ccols replaces C/ldc.
  const void* const* bcols = nullptr;
  void* const* ccols = nullptr;
  // A (op_a N only) by the bases of its k stored columns of m elements; replaces A/lda.
  const void* const* acols = nullptr;
  // Set by the grouped entry point: whether every column base allows 16-byte
  // loads (B) and 4-element vector stores (C).
  bool cols_vec_ld = false;
  bool cols_vec_c = false;
  // The tables themselves sit in the context workspace, so split-K, which
  // keeps its partial sums there, is not available.
  bool cols_in_workspace = false;
};

// Validates shapes and enqueues the product on ctx->stream.
int launch_gemm(ginn_hip_ctx* ctx, const GemmArgs& args);

// Generic LDS-tiled MFMA kernel for any shape / alignment.
int launch_gemm_generic(ginn_hip_ctx* ctx, const GemmArgs& args);

// Tuned kernel for large, aligned fp16 / bf16 products; returns kUnsupported
// (without setting an error) when the shape does not qualify.
int launch_gemm_fast16(ginn_hip_ctx* ctx, const GemmArgs& args);

// fp32 products with at most a few hundred 32 x 32 output tiles: K split over
// the 16 waves of a workgroup, one launch; kUnsupported otherwise.
int launch_gemm_ksplit(ginn_hip_ctx* ctx, const GemmArgs& args);

// Element-wise arithmetic on 32-bit integer tensors (GINN_HIP_I32), exact: dst (+)= op(a, b, c).
// kIntAdd: a + b (b may be NULL); kIntScaleShift: ia * a + ib; kIntMulAdd: a (*) (b + ia) + c with b and c
// indexed per row (i % rows) when rows != 0.
enum IntOp { kIntAdd = 0, kIntSub, kIntMul, kIntMax, kIntScaleShift, kIntMulAdd };
int launch_int_arith(ginn_hip_ctx* ctx, int op, size_t n, size_t rows, const void* a, const void* b, const void* c,
                     int ia, int ib, void* dst, int accumulate);
// Select, Mask (forward, no accumulation) and UpperTri on 32-bit integers; operands checked by the callers.
int launch_int_select(ginn_hip_ctx* ctx, size_t n, const unsigned char* cond, const void* a, int a_is_scalar,
                      const void* b, int b_is_scalar, void* dst);
int launch_int_mask(ginn_hip_ctx* ctx, size_t mask_size, size_t n, const void* mask, int value, const void* x,
                    void* dst);
int launch_int_upper_tri(ginn_hip_ctx* ctx, size_t n, void* dst);
// Bandwidth-oriented kernel for narrow right-hand sides (n <= 64).
int launch_gemm_skinny(ginn_hip_ctx* ctx, const GemmArgs& args);
int launch_gemm_strip(ginn_hip_ctx* ctx, const GemmArgs& args);
int launch_gemm_skinny_mfma(ginn_hip_ctx* ctx, const GemmArgs& args);
// 16-bit, 128 x 128 x 64 tiles with optional split-K: aligned shapes whose
// 256 x 256 tiling would leave most CUs idle; kUnsupported otherwise.
int launch_gemm_mid(ginn_hip_ctx* ctx, const GemmArgs& args);
// Batched 16-bit products with small, memory-bound slices (attention shapes);
// kUnsupported for everything else (gemm_bsmall.hip).
int launch_gemm_bsmall(ginn_hip_ctx* ctx, const GemmArgs& args);
// Folds `splits` fp32 partial products [split][n][m] and applies the epilogue
// of `args` (beta, bias, activation, pre-activation) into C.
int launch_splitk_reduce(ginn_hip_ctx* ctx, const GemmArgs& args, int splits, const float* partial);

// Looks up, once per GPU and with that GPU current, the device address of the
// scratch array behind ginn_hip_gemm_noalloc.
void noalloc_prepare(int device);

int launch_softmax_fwd(ginn_hip_ctx* ctx, int dtype, int rows, int cols,
                       const void* x, void* y);

// Uploads `bytes` from host memory into the context workspace at `offset`
// through the pinned staging ring; the copy is ordered on ctx->stream.
int stage_to_workspace(ginn_hip_ctx* ctx, size_t offset, const void* host_src,
                       size_t bytes);

}  // namespace ginn_hip

#endif  // GINN_HIP_COMMON_H
