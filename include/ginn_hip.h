/*
 * ginn_hip.h -- C ABI of libginn_hip.so, the MI355X (gfx950) device layer and
 * matrix-product kernels behind GINN's `ginn::internal::gpu_prod` /
 * `gpu_batched_prod`, `ProdNode`, `BatchedProdNode` and `AffineNode`.
 *
 * Conventions
 *  - Every matrix is COLUMN-MAJOR with an explicit leading dimension, exactly
 *    as the reference hands them to its BLAS (ginn/prod.h:211-253).
 *  - Every function returns 0 on success and a non-zero status otherwise; the
 *    message for the calling thread's last failure is ginn_hip_last_error().
 *    No C++ exception crosses this boundary.
 *  - All work is enqueued on the context's single stream.  Only
 *    ginn_hip_memcpy_d2h and ginn_hip_sync block the host.
 *  - Pointers named A, B, C, W, X, Y, bias, ... are DEVICE pointers unless
 *    the parameter name starts with `host_`.
 *  - The library never falls back to a host computation: an unsupported
 *    argument is an error.
 */
#ifndef GINN_HIP_H
#define GINN_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Opaque per-device context: one device index, one stream, one workspace.
 * Replaces GpuDevice's {cudaStream_t, cublasHandle_t} pair
 * (ginn/dev.h:149-199) and the `cublas_handle(idx)` accessor
 * (ginn/dev.h:264). */
typedef struct ginn_hip_ctx ginn_hip_ctx;

/* Bump-pointer device arena; replaces PreallocGpuDevice
 * (ginn/dev.h:214-254). */
typedef struct ginn_hip_arena ginn_hip_arena;

/* Scalar types of the path.  F32 = ginn::Real, F16 = ginn::Half
 * (ginn/def.h:31-39).  BF16 has no counterpart in the reference; it is bit
 * pattern "upper 16 bits of an IEEE float". */
typedef enum ginn_hip_dtype {
  GINN_HIP_F32 = 0,
  GINN_HIP_F16 = 1,
  GINN_HIP_BF16 = 2,
  /* ginn::Int tensors (indices, conditions): accepted only where a declaration
   * says so -- the comparison, and the forward arithmetic of the nodes the
   * reference instantiates on Int (ginn_hip_add_n, _cwise_prod, _scale_shift,
   * _elementwise SUB / MAX, _cwise_prod_add_fwd), exact and wrapping. */
  GINN_HIP_I32 = 3
} ginn_hip_dtype;

/* CUBLAS_OP_N / CUBLAS_OP_T as used by ginn/prod.h:217-222. */
typedef enum ginn_hip_op { GINN_HIP_OP_N = 0, GINN_HIP_OP_T = 1 } ginn_hip_op;

/* Nonlinearities that AffineNode can carry (ginn/nonlin.h:67-300).
 * SOFTMAX is column-wise and is never fused into a GEMM tile; LOG and SQRT
 * exist for the stand-alone nonlinearity entry points only. */
typedef enum ginn_hip_act {
  GINN_HIP_ACT_IDENTITY = 0,
  GINN_HIP_ACT_TANH = 1,
  GINN_HIP_ACT_RELU = 2,
  GINN_HIP_ACT_SIGMOID = 3,
  GINN_HIP_ACT_GELU = 4,  /* erf form,  ginn/nonlin.h:273-300 */
  GINN_HIP_ACT_GELU2 = 5, /* tanh form, ginn/nonlin.h:242-271 */
  GINN_HIP_ACT_SOFTMAX = 6,
  GINN_HIP_ACT_LOG = 7,
  GINN_HIP_ACT_SQRT = 8
} ginn_hip_act;

/* ------------------------------------------------------------------ */
/* Errors                                                              */
/* ------------------------------------------------------------------ */

/* Message of the last failing call on this thread ("" if none).  Plays the
 * role of the text carried by ginn::CudaError (ginn/cudef.h:23-59). */
const char* ginn_hip_last_error(void);

/* ------------------------------------------------------------------ */
/* Device / context  (ginn/dev.h:38-46, 149-212)                       */
/* ------------------------------------------------------------------ */

/* Number of visible GPUs; replaces ginn::gpus() (ginn/dev.h:38-46). */
int ginn_hip_device_count(int* count);

/* Creates a context on `device` with a stream of its own (default priority)
 * and a workspace of `workspace_bytes` (0 = default, 64 MiB); replaces the
 * GpuDevice constructor (ginn/dev.h:183-192). */
int ginn_hip_ctx_create(int device, size_t workspace_bytes, ginn_hip_ctx** ctx);

/* Same, but enqueues on an existing hipStream_t that the caller owns
 * (`stream` may be NULL for the device's null stream). */
int ginn_hip_ctx_create_on_stream(int device, void* stream,
                                  size_t workspace_bytes, ginn_hip_ctx** ctx);

/* Destroys the context; replaces ~GpuDevice (ginn/dev.h:194-198). */
int ginn_hip_ctx_destroy(ginn_hip_ctx* ctx);

/* Device index and hipStream_t of the context (GpuDevice::id / ::stream,
 * ginn/dev.h:176-177). */
int ginn_hip_ctx_device(const ginn_hip_ctx* ctx, int* device);
int ginn_hip_ctx_stream(const ginn_hip_ctx* ctx, void** stream);

/* Orders two contexts of one device: what is enqueued on `waiter` after this
 * call runs after everything enqueued on `signaler` before it (an event
 * recorded on one stream and waited for on the other; the host does not
 * wait).  With it work that nothing on a context's stream depends on can run
 * beside that stream on a second context and be joined later: the drop-in
 * headers run the products into the gradients of weights (leaves, complete
 * only when the backward pass ends: ginn/node/prod.h:57-63,
 * ginn/node/affine.h:117-122) that way, so they share the device with the
 * chain of launches every other node waits for instead of each taking its
 * turn with a part of it.  The reference has one handle and the legacy
 * default stream (ginn/dev.h:188-189).  *ordered is set to 0, and nothing is
 * enqueued, while either stream is recording a device graph: the caller then
 * keeps the work on one context. */
int ginn_hip_ctx_wait_for(ginn_hip_ctx* waiter, ginn_hip_ctx* signaler,
                          int* ordered);

/* Blocks until the context's stream is idle (cudaStreamSynchronize /
 * cudaDeviceSynchronize as used in ginn/util/timer.h:36-45). */
int ginn_hip_sync(ginn_hip_ctx* ctx);

/* ------------------------------------------------------------------ */
/* Memory  (ginn/dev.h:158-175, 269-343)                               */
/* ------------------------------------------------------------------ */

/* GpuDevice::alloc / ::free (ginn/dev.h:158-175).  Where the reference calls
 * cudaMalloc / cudaFree per temporary tensor, released blocks are kept by the
 * context (sizes rounded to powers of two up to 2 MiB, to multiples of 2 MiB
 * above) and handed out again without a driver call.  That is safe because a
 * context's memory is only used on its one stream: whatever still reads a
 * released block was enqueued before the block's next user.  Memory obtained
 * here must not be used on another stream without the caller's own ordering.
 * Blocks of up to 64 KiB are cut, in address order, from 2 MiB driver
 * allocations of their size class, which go back to the driver when none of
 * their blocks is in use and the cache is emptied or over its bound: a graph
 * of many small tensors costs few driver calls and its tensors share pages. */
int ginn_hip_malloc(ginn_hip_ctx* ctx, size_t bytes, void** ptr);
int ginn_hip_free(ginn_hip_ctx* ctx, void* ptr);
/* The cache of released blocks: switch it off (enabled = 0: malloc / free go to
 * the driver as in the reference), bound it (default 8 GiB; blocks released
 * beyond the bound go back to the driver), empty it (waits for the stream), or
 * read it (bytes held for reuse, and blocks the pool knows, in use or held). */
int ginn_hip_pool_configure(ginn_hip_ctx* ctx, int enabled, size_t limit_bytes);
int ginn_hip_pool_trim(ginn_hip_ctx* ctx);
/* The most device memory ONE product (ginn_hip_gemm, ginn_hip_affine_fwd) may take from
 * ginn_hip_malloc for copies of operands whose leading dimensions or addresses rule out
 * 16-byte accesses (default 2 GiB; 0: products never allocate).  cuBLAS takes such
 * operands in place (ginn/prod.h:46-62); here a large product on them runs on padded
 * copies when they fit the budget and the device has the room, and in place on the
 * any-shape kernel otherwise -- a product never fails for want of that memory.  The
 * blocks go back to the context's cache of released blocks after the call. */
int ginn_hip_gemm_temp_budget(ginn_hip_ctx* ctx, size_t bytes);
int ginn_hip_pool_stats(ginn_hip_ctx* ctx, size_t* cached_bytes, size_t* blocks);

/* Device::copy, GPU<-CPU branch: asynchronous on the stream
 * (ginn/dev.h:276-280).  `host_src` must stay valid until the stream reaches
 * the copy. */
int ginn_hip_memcpy_h2d(ginn_hip_ctx* ctx, void* dst, const void* host_src,
                        size_t bytes);
/* Device::copy, CPU<-GPU branch: blocks until the bytes are in `host_dst`
 * (ginn/dev.h:273-275). */
int ginn_hip_memcpy_d2h(ginn_hip_ctx* ctx, void* host_dst, const void* src,
                        size_t bytes);
/* Device::copy, same-GPU branch (ginn/dev.h:282-287). */
int ginn_hip_memcpy_d2d(ginn_hip_ctx* ctx, void* dst, const void* src,
                        size_t bytes);
/* Byte fill on the stream (Tensor::set_zero on a GPU tensor,
 * ginn/tensor.h:442). Implemented as a kernel so that it can be captured. */
int ginn_hip_memset(ginn_hip_ctx* ctx, void* dst, int byte_value, size_t bytes);

/* PreallocGpuDevice (ginn/dev.h:214-254): one slab, bump allocation, no
 * per-allocation free, clear() rewinds.  As in the reference an allocation
 * must leave at least one byte unused (`<`, not `<=`, ginn/dev.h:238-241),
 * and as there the bump is byte-exact: used() is the sum of the sizes asked
 * for, and a block starts where the last one ended (the slab itself is
 * 256-byte aligned).  Every kernel of this library takes operands at any
 * element-aligned address and falls back from 16-byte to element accesses
 * when a pointer is not 16-byte aligned. */
int ginn_hip_arena_create(ginn_hip_ctx* ctx, size_t bytes,
                          ginn_hip_arena** arena);
int ginn_hip_arena_destroy(ginn_hip_arena* arena);
int ginn_hip_arena_alloc(ginn_hip_arena* arena, size_t bytes, void** ptr);
int ginn_hip_arena_clear(ginn_hip_arena* arena);
/* No counterpart in the reference: from now on every block starts at a
 * multiple of `alignment` bytes (a power of two <= 4096; 1 restores the
 * byte-exact bump), so that tensors of mixed scalar types stay aligned and
 * the 16-byte access paths are taken; the padding counts as used. */
int ginn_hip_arena_set_alignment(ginn_hip_arena* arena, size_t alignment);
int ginn_hip_arena_used(const ginn_hip_arena* arena, size_t* bytes);
int ginn_hip_arena_size(const ginn_hip_arena* arena, size_t* bytes);

/* ------------------------------------------------------------------ */
/* Matrix products  (ginn/prod.h:32-135)                               */
/* ------------------------------------------------------------------ */

/* C[m x n] = op(A)[m x k] * op(B)[k x n] + beta * C, alpha fixed to 1;
 * replaces gpu_gemm -> cublasSgemm / cublasHgemm (ginn/prod.h:32-66).
 * fp16 / bf16 operands are multiplied exactly and accumulated in fp32; the
 * result is rounded to the storage type once (twice where a large product
 * with extents that are no multiples of the kernels' tiles is cut into a
 * tuned core and a rest).  beta == 0 never reads C.  A large product whose
 * leading dimensions or pointers rule out 16-byte accesses is computed on
 * copies with padded leading dimensions, in blocks of the context's pool
 * (ginn_hip_malloc / ginn_hip_free); not while the stream is captured. */
int ginn_hip_gemm(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, ginn_hip_op op_a,
                  ginn_hip_op op_b, int m, int n, int k, const void* A,
                  int lda, const void* B, int ldb, float beta, void* C,
                  int ldc);

/* `batch` products of identical shape, operand i at base + i * stride
 * (element counts); replaces gpu_batched_gemm -> cublas?gemmStridedBatched
 * (ginn/prod.h:68-135). */
int ginn_hip_gemm_strided_batched(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                  ginn_hip_op op_a, ginn_hip_op op_b, int m,
                                  int n, int k, const void* A, int lda,
                                  long long stride_a, const void* B, int ldb,
                                  long long stride_b, float beta, void* C,
                                  int ldc, long long stride_c, int batch);

/* The same with the slices numbered in two levels: slice z, z < batch_inner *
 * batch_outer, of an operand lies at base + (z % batch_inner) * stride +
 * (z / batch_inner) * stride2.  This is how the [rows x cols] slices of a
 * rank-4 tensor lie in memory AFTER a permutation of its axes that keeps (or
 * swaps) the first two: BatchedProdNode (ginn/node/prod.h:104-187) reads the
 * heads of an attention layer where the projection wrote them, and writes its
 * result where the next projection reads it, instead of through PermuteNode
 * copies (ginn/node/layout.h:723-821; examples/min-gpt.cu.cpp:117-135).  One
 * launch where the small-slice kernel takes the shape, batch_outer strided
 * batches otherwise. */
int ginn_hip_gemm_strided_batched2(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                   ginn_hip_op op_a, ginn_hip_op op_b, int m,
                                   int n, int k, const void* A, int lda,
                                   long long stride_a, long long stride_a2,
                                   const void* B, int ldb, long long stride_b,
                                   long long stride_b2, float beta, void* C,
                                   int ldc, long long stride_c,
                                   long long stride_c2, int batch_inner,
                                   int batch_outer);

/* ginn_hip_gemm for callers that cannot allocate: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no
 * counterpart in the reference (whose BLAS handle allocates its workspace
 * when it is created, ginn/dev.h:188-189).  Same product, same kernels; it
 * takes a device index and a hipStream_t (NULL = the null stream) instead of
 * a context, and the split-K partial sums live in a 16 MiB device array that
 * is part of the library image (one copy per GPU, held until the process
 * ends).  The call allocates and frees nothing: no hipMalloc, hipHostMalloc
 * or hipFree, no context.
 * Limit: m * n <= 2 097 152 output elements (two fp32 partial copies of the
 * output fit the array) -- the small and skinny products of a serving loop;
 * a larger output is refused with an error, use ginn_hip_gemm for it.
 * All calls on one GPU share that GPU's array: calls that overlap in time on
 * one GPU (two streams, or two processes' worth of graphs replayed at once)
 * race on it; calls on one stream, or on streams the caller orders, do not.
 * The array's old contents never matter (partial sums are written before
 * they are read).  The address of the array is looked up once per GPU, at
 * the first ginn_hip_ctx_create on that GPU or at the first call of this
 * function, whichever comes first: make that first use outside a capture. */
int ginn_hip_gemm_noalloc(int device, void* stream, ginn_hip_dtype dtype,
                          ginn_hip_op op_a, ginn_hip_op op_b, int m, int n,
                          int k, const void* A, int lda, const void* B,
                          int ldb, float beta, void* C, int ldc);

/* One launch for `groups` products that share the left operand:
 * C_g[m x n_g] = op(A) * B_g[k x n_g] + beta * C_g.  This is the product
 * that Autobatch forms by concatenating right-hand sides
 * (ginn/autobatch.h:149-183, ginn/node/layout.h:221-315) without the
 * concatenation copy.  The four tables are HOST arrays of length `groups`;
 * the library stages them through its workspace. */
int ginn_hip_gemm_grouped(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                          ginn_hip_op op_a, int m, int k, const void* A,
                          int lda, int groups, const void* const* host_B,
                          const int* host_n, const int* host_ldb, float beta,
                          void* const* host_C, const int* host_ldc);

/* A product whose right operand and / or output live in scattered columns:
 * C[m x n] = op(A)[m x k] * op(B)[k x n] + beta * C, where
 *   dev_b_cols, when not NULL, replaces (B, ldb): a DEVICE table holding the
 *     base of every stored column of B -- n entries of k elements when op_b
 *     is N, k entries of n elements when op_b is T;
 *   dev_c_cols, when not NULL, replaces (C, ldc): a DEVICE table of n column
 *     bases of m elements.
 * With it the merged product of Autobatch (ginn/autobatch.h:149-183) reads
 * the right operands where they are (op_b N), adds their gradients where
 * they are (op_a T, dev_c_cols) and forms the gradient of the shared left
 * operand as a sum over all their columns (op_b T), so neither RowwiseCat's
 * copy nor its backward (ginn/node/layout.h:221-315) runs.  The tables stay
 * valid across calls as long as the operands do not move; the caller owns
 * them.  cols_aligned != 0 promises 16-byte aligned column bases (then
 * 16-byte accesses are used when the extents allow). */
int ginn_hip_gemm_gathered(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                           ginn_hip_op op_a, ginn_hip_op op_b, int m, int n,
                           int k, const void* A, int lda, const void* B,
                           int ldb, const void* const* dev_b_cols, float beta,
                           void* C, int ldc, void* const* dev_c_cols,
                           int cols_aligned);

/* C[m x n] = sum_{j < k} a_j b_j^T + beta * C: a sum of outer products of
 * scattered columns, a_j (m elements) at dev_a_cols[j], b_j (n elements) at
 * dev_b_cols[j]; both tables are DEVICE arrays of k entries.  A shared left
 * operand W of several products Y_t = W X_t receives dW += dY_t X_t^T from
 * each of them (ProdNode::backward_, ginn/node/prod.h:57-63; for the products
 * Autobatch merges, ginn/autobatch.h:149-183, once per merged group): with
 * the columns of all dY_t and all X_t listed in the two tables this is ONE
 * product that sums over every column of every use, run once at the end of
 * the backward pass.  cols_aligned != 0 promises 16-byte aligned column
 * bases.  C is dense (ldc >= m). */
int ginn_hip_gemm_outer_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int m,
                            int n, int k, const void* const* dev_a_cols,
                            const void* const* dev_b_cols, float beta,
                            void* C, int ldc, int cols_aligned);

/* out[c] = sum_r x[r, c] * y[r, c] + beta * out[c] for `cols` columns of
 * height `rows` (contiguous, ld = rows).  This is the degenerate m = n = 1
 * batched product that SoftmaxOp::backward (ginn/nonlin.h:177-184) and
 * LayerNormNode::backward_ (ginn/node/layernorm.h:60-64) issue; the batched
 * entry point above routes that shape here. */
int ginn_hip_col_dot_batched(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                             int cols, const void* x, const void* y,
                             float beta, void* out);

/* ------------------------------------------------------------------ */
/* AffineNode  (ginn/node/affine.h:35-129)                             */
/* ------------------------------------------------------------------ */

/* Y[m x n] = act( sum_p W_p[m x k_p] * X_p[k_p x n] + bias[m] ), bias
 * broadcast along columns; replaces AffineNode::forward_
 * (ginn/node/affine.h:35-77): bias broadcast kernel + one beta=1 GEMM per
 * pair + the activation kernels become the epilogue of the last GEMM.
 * `pre` (ld = m) receives the pre-activation when it is not NULL -- pass it
 * exactly when the activation's backward needs its input (GELU, GELU2,
 * SOFTMAX; ginn/node/affine.h:44-46).  The per-pair tables are HOST arrays
 * of length `pairs`.  Y and pre are dense (ld = m).  SOFTMAX runs as a
 * second, column-wise kernel after the GEMM. */
int ginn_hip_affine_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int m, int n, int pairs,
                        const void* const* host_W, const void* const* host_X,
                        const int* host_k, const void* bias, void* pre,
                        void* Y);

/* First half of AffineNode::backward_ (ginn/node/affine.h:80-93,107):
 * dpre = act'(.) (*) dY and dbias[m] += sum_cols dpre in one pass.  For
 * IDENTITY dpre is not written (the caller uses dY itself) and only the
 * bias gradient is accumulated.  `pre` may be NULL when the activation's
 * backward does not need it; `dbias` may be NULL when the bias has no
 * gradient.  The two accumulating GEMMs per pair that follow
 * (ginn/node/affine.h:110-123) are plain ginn_hip_gemm calls. */
int ginn_hip_affine_bwd_pre(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                            ginn_hip_act act, int m, int n, const void* dY,
                            const void* Y, const void* pre, void* dpre,
                            void* dbias);

/* ------------------------------------------------------------------ */
/* Stand-alone nonlinearities  (ginn/nonlin.h:42-300)                  */
/* ------------------------------------------------------------------ */

/* y = act(x) over a dense [rows x cols] matrix; NonlinOp::forward.
 * SOFTMAX normalises down each column (ginn/nonlin.h:162-168). */
int ginn_hip_nonlin_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int rows, int cols, const void* x,
                        void* y);

/* dx (+)= act'(x, y) (*) dy; NonlinOp::backward with its `accumulate` flag
 * (ginn/nonlin.h:52-57).  `x` may be NULL when the op does not need it. */
int ginn_hip_nonlin_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                        ginn_hip_act act, int rows, int cols, const void* dy,
                        const void* x, const void* y, void* dx,
                        int accumulate);

/* ------------------------------------------------------------------ */
/* Data-movement and elementwise companions of the product path.       */
/* The reference evaluates these as Eigen expressions on its GPU       */
/* device (ginn/tensor.h:616-628); here each is one small kernel.      */
/* ------------------------------------------------------------------ */

/* dst[0..n) = value; Tensor::fill (ginn/tensor.h:442-446). */
int ginn_hip_fill(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, void* dst, size_t n,
                  float value);

/* dst (+)= src over a [rows x cols] column-major window with leading
 * dimensions lds / ldd: the slice assignments of Cat, RowwiseCat, Slice and
 * their `+=` backward forms (ginn/node/layout.h:175-198,227-253,566-577). */
int ginn_hip_copy_2d(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                     int cols, const void* src, int lds, void* dst, int ldd,
                     int accumulate);

/* dst (+)= src_0 + ... + src_{count-1}, n elements each; AddNode forward
 * and the `grad() += ...` of every backward (ginn/node/common.h:116-139).
 * host_srcs is a HOST array of `count` (1..8) device pointers.  dtype may be
 * GINN_HIP_I32 (Add on Int, test/nodes.cu.cpp:443-487). */
int ginn_hip_add_n(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n, int count,
                   const void* const* host_srcs, void* dst, int accumulate);

/* dst (+)= a (*) b elementwise; CwiseProdNode forward / backward
 * (ginn/node/common.h:233-262).  dtype may be GINN_HIP_I32. */
int ginn_hip_cwise_prod(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                        const void* a, const void* b, void* dst,
                        int accumulate);

/* dst (+)= alpha * x + shift; ProdScalar / AddScalar and their backward
 * (ginn/node/common.h:32-95,187-231).  dtype may be GINN_HIP_I32: alpha and
 * shift are then truncated to integers (the node holds them as Int). */
int ginn_hip_scale_shift(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                         float alpha, float shift, const void* x, void* dst,
                         int accumulate);

/* dst[r, c] = x[r] for c < cols; ColBroadcastNode forward and the bias
 * broadcast of AffineNode (ginn/node/layout.h:869-881, ginn/node/affine.h:57). */
int ginn_hip_col_broadcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                           int cols, const void* x, void* dst);

/* dst[r] (+)= sum_c x[r, c]; ColBroadcast backward and the bias gradient
 * (ginn/node/layout.h:883-887, ginn/node/affine.h:107). */
int ginn_hip_row_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols,
                     const void* x, void* dst, int accumulate);

/* Row sums are two launches: partial sums per chunk of columns, then a fold of
 * the chunks.  A backward pass makes one such pair per bias gradient
 * (AffineNode::backward_, ginn/node/affine.h:117-122) and per scale / shift
 * gradient of CwiseProdAdd (ginn/node/common.h:296-316); the reference does
 * each as one Eigen reduction.  A caller that does not read those sums before
 * the end of the pass may postpone the folds and run them as one launch:
 *   ginn_hip_defer_folds(ctx, 1);   folds of row reductions that THIS host
 *                                   thread starts from now on are queued
 *                                   (ginn_hip_affine_bwd_pre's dbias,
 *                                   ginn_hip_cwise_prod_add_bwd's db / dc,
 *                                   ginn_hip_row_sum); calls nest
 *   ginn_hip_defer_folds(ctx, 0);   back to folding at once (queued folds stay queued)
 *   ginn_hip_flush_folds(ctx);      one launch for everything queued on ctx
 * Until the flush the destinations hold their old values.  The queue also
 * empties by itself when its 8 MiB of partial sums are full, when two queued
 * folds would add into one destination, and in ginn_hip_sync.  The sums are
 * the same bits as without postponing. */
int ginn_hip_defer_folds(ginn_hip_ctx* ctx, int on);
int ginn_hip_flush_folds(ginn_hip_ctx* ctx);
int ginn_hip_pending_folds(ginn_hip_ctx* ctx, int* count);

/* dst[0] = scale * sum_i x[i]; SumNode / MeanNode forward
 * (ginn/node/reduce.h:30-75,138-159). */
int ginn_hip_sum_all(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                     const void* x, float scale, void* dst);

/* dst[i] += scale * src[0]; SumNode / MeanNode backward. */
int ginn_hip_add_scalar_bcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                              const void* src, float scale, void* dst);

/* PickNegLogSoftmaxNode (ginn/node/pick.h:178-236): smax = column softmax of
 * x [rows x cols]; out[c] = -log smax[idx[c], c].  idx is a DEVICE array of
 * `cols` int32 row indices. */
int ginn_hip_pick_nls_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                          int cols, const void* x, const int* idx, void* smax,
                          void* out);
/* dx[:, c] += smax[:, c] * dout[c]; dx[idx[c], c] -= dout[c]. */
int ginn_hip_pick_nls_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                          int cols, const void* smax, const int* idx,
                          const void* dout, void* dx);
/* The pair without the softmax matrix: forward leaves stats[2 c] = maximum of
 * column c and stats[2 c + 1] = 1 / sum_r exp(x[r, c] - maximum) (fp32, DEVICE
 * array of 2 * cols), backward rebuilds softmax(x) from them, rounded to the
 * storage type as ginn_hip_pick_nls_fwd would have stored it, and assigns
 * (accumulate == 0) or adds.  x must still hold the forward pass's values. */
int ginn_hip_pick_nls_fwd_stats(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                int rows, int cols, const void* x,
                                const int* idx, float* stats, void* out);
int ginn_hip_pick_nls_bwd_stats(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                int rows, int cols, const void* x,
                                const float* stats, const int* idx,
                                const void* dout, void* dx, int accumulate);
/* The same with `=` in place of `+=`: what the backward pass of
 * ginn/node/pick.h:226-236 leaves in a gradient that reset_grad() had just
 * zeroed (ginn/node.h:218-222), without reading the zeros. */
int ginn_hip_pick_nls_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                 int rows, int cols, const void* smax,
                                 const int* idx, const void* dout, void* dx);

/* ------------------------------------------------------------------ */
/* Transformer-block companions (column-major, fp32 statistics)        */
/* ------------------------------------------------------------------ */

/* LayerNormNode::forward_ (ginn/node/layernorm.h:31-47): per column of
 * x [rows x cols], y = (x - mean) / std with std = sqrt(mean((x-mean)^2) + eps).
 * std_out is a DEVICE array of `cols` floats kept for the backward pass. */
int ginn_hip_layernorm_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                           int cols, const void* x, float eps, void* y,
                           float* std_out);
/* LayerNormNode::backward_ (ginn/node/layernorm.h:49-74), including the
 * per-column dot product the reference computes with a degenerate batched
 * gemm: dx += (dy - mean(dy) - y * (dy . y) / rows) / std. */
int ginn_hip_layernorm_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                           int cols, const void* dy, const void* y,
                           const float* std_in, void* dx);

/* CwiseProdAddNode (ginn/node/common.h:251-296): y = a * (b + multiplier_bias)
 * + c.  With broadcast != 0, b and c are [rows] vectors applied to every
 * column of a [rows x cols] (the LayerNorm gamma / beta form).  dtype may be
 * GINN_HIP_I32 (forward only). */
int ginn_hip_cwise_prod_add_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                int rows, int cols, const void* a,
                                const void* b, const void* c,
                                float multiplier_bias, int broadcast, void* y);
/* Accumulates into whichever of da, db, dc is not NULL; with broadcast, db
 * and dc are row sums over the columns. */
int ginn_hip_cwise_prod_add_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                int rows, int cols, const void* dy,
                                const void* a, const void* b,
                                float multiplier_bias, int broadcast, void* da,
                                void* db, void* dc);
/* The same with da assigned instead of added to (a gradient that reset_grad()
 * had just zeroed, ginn/node.h:218-222); db and dc are added to as above. */
int ginn_hip_cwise_prod_add_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                       int rows, int cols, const void* dy,
                                       const void* a, const void* b,
                                       float multiplier_bias, int broadcast,
                                       void* da, void* db, void* dc);

/* LayerNorm followed by the gamma / beta step, z = LayerNorm(x) * (gamma +
 * multiplier_bias) + beta with gamma, beta [rows] vectors: the pair
 * LayerNormNode (ginn/node/layernorm.h:31-47) + CwiseProdAddNode
 * (ginn/node/common.h:251-296) of examples/min-gpt.cu.cpp:100-103 as one pass.
 * y [rows x cols] receives the normalised values and std_out [cols] the
 * statistics, as ginn_hip_layernorm_fwd leaves them (both are needed for the
 * backward pass); z is computed from y as stored.  Same bits as the two
 * separate calls. */
int ginn_hip_layernorm_affine_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                  int rows, int cols, const void* x, float eps,
                                  const void* gamma, const void* beta,
                                  float multiplier_bias, void* y,
                                  float* std_out, void* z);
/* Backward of the pair for a gradient of y that holds no value yet (y has no
 * other user): dx (+)= LayerNorm backward of da = dz * (gamma +
 * multiplier_bias), da rounded to the storage type but never stored;
 * dgamma += sum_c dz (*) y, dbeta += sum_c dz (both or neither; their fold can
 * be postponed, see ginn_hip_defer_folds).  dx may be NULL; accumulate == 0
 * assigns dx.  Results as from ginn_hip_cwise_prod_add_bwd_assign followed by
 * ginn_hip_layernorm_bwd(_assign) up to fp32 rounding (the compiler contracts
 * the same expressions differently in the two kernels; the row sums are taken
 * in another order of the columns). */
int ginn_hip_layernorm_affine_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                  int rows, int cols, const void* dz,
                                  const void* y, const float* std_in,
                                  const void* gamma, float multiplier_bias,
                                  void* dx, int accumulate, void* dgamma,
                                  void* dbeta);

/* PermuteNode (ginn/node/layout.h:723-821): dst has extents
 * dims[perm[0]], dims[perm[1]], ... and dst[i_perm] = src[i] (Eigen's
 * shuffle).  dims / perm are HOST arrays of `rank` (<= 8) entries;
 * accumulate != 0 adds into dst (the backward pass with the inverse perm). */
int ginn_hip_permute(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank,
                     const long long* host_dims, const int* host_perm,
                     const void* src, void* dst, int accumulate);

/* InPlaceMaskNode (ginn/node/inplace.h:152-196): x viewed as
 * [mask_size x batch]; entries whose mask value is 0 become `value` (forward:
 * the mask value, e.g. -inf; backward: 0 on the gradient). */
int ginn_hip_mask_fill(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                       size_t mask_size, size_t batch, const void* mask,
                       float value, void* x);

/* The score chain of an attention block as one pass: InPlaceProdScalar
 * (ginn/node/inplace.h:104-123), InPlaceMask (:152-212) and Softmax
 * (ginn/nonlin.h:162-168) over x [rows x cols], softmax down the columns.
 *   x <- scale * x;  x[i] <- fill where mask[i % mask_n] == 0;  y = softmax(x)
 * x is updated in place, as the two in-place nodes leave it; y is a different
 * array.  mask has the operand's dtype and mask_n divides rows * cols.  Every
 * step rounds to the storage type like the separate calls (ginn_hip_scale_shift,
 * ginn_hip_mask_fill, ginn_hip_nonlin_fwd) do: same bits, one read of x. */
int ginn_hip_scaled_masked_softmax_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                       int rows, int cols, void* x, float scale,
                                       const void* mask, size_t mask_n,
                                       float fill, void* y);
/* The three backward steps (ginn/nonlin.h:170-188, ginn/node/inplace.h:198-212
 * and :118-122) for a gradient that holds no value yet:
 *   dx = scale * (mask ? y (*) (dy - colsum(y (*) dy)) : 0), assigned. */
int ginn_hip_scaled_masked_softmax_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                       int rows, int cols, const void* dy,
                                       const void* y, float scale,
                                       const void* mask, size_t mask_n,
                                       void* dx);

/* UpperTriNode (ginn/node/layout.h:922-955): dst [n x n] = 1 where
 * row <= col, else 0.  dtype may be GINN_HIP_I32. */
int ginn_hip_upper_tri(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int n,
                       void* dst);

/* LayerNormNode::backward_ of the in-place node (ginn/node/inplace.h:214-246):
 * dx = (...) / std, assigned; dx may be dy itself. */
int ginn_hip_layernorm_bwd_assign(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                                  int rows, int cols, const void* dy,
                                  const void* y, const float* std_in, void* dx);

/* ------------------------------------------------------------------ */
/* The other nodes around the products: arithmetic, selection, gather  */
/* / scatter, reductions, random fills.  Eigen expressions, thrust      */
/* gathers and the two Stack kernels in the reference.                  */
/* ------------------------------------------------------------------ */

typedef enum {
  GINN_HIP_EW_SUB = 0,    /* a - b                 SubtractNode forward (ginn/node/common.h:162-187) */
  GINN_HIP_EW_MAX = 1,    /* max(a, b)             CwiseMaxNode forward, pairwise (:319-330) */
  GINN_HIP_EW_EQ_MUL = 2, /* a * (b == c ? 1 : 0)  CwiseMaxNode backward (:332-341) */
  GINN_HIP_EW_DIV_MUL = 3 /* a * (b / c)           InPlaceCwiseProdNode backward (ginn/node/inplace.h:88-93) */
} ginn_hip_ew_op;

/* dst (+)= op(a, b, c) over n elements; c is read by the three-operand forms
 * only.  dst may be one of the operands.  SUB and MAX also take GINN_HIP_I32. */
int ginn_hip_elementwise(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                         ginn_hip_ew_op op, size_t n, const void* a,
                         const void* b, const void* c, void* dst,
                         int accumulate);

/* U[lo, hi) fill: element i is a function of (seed, i) alone.  Replaces
 * curandGenerateUniform + `-1 + 2 x` of Tensor::set_random on a GPU tensor
 * (ginn/tensor.h:459-462, ginn/cudef.h:63-89); the value stream differs from
 * cuRAND's, as cuRAND's differs from Eigen's. */
int ginn_hip_fill_uniform(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                          unsigned long long seed, float lo, float hi,
                          void* dst);

/* DropoutNode (ginn/node/common.h:359-402): mask[i] = (u_i >= p), one byte
 * per element, u_i uniform in [0, 1) from (seed, i); then
 * dst (+)= x * mask * scale with scale = 1 / (1 - p) serves the forward pass
 * and, on the gradient, the backward pass (dst may be x: InPlaceDropout,
 * ginn/node/inplace.h:126-150). */
int ginn_hip_dropout_mask(ginn_hip_ctx* ctx, size_t n, float p,
                          unsigned long long seed, unsigned char* mask);
int ginn_hip_mask_scale(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                        float scale, const void* x, const unsigned char* mask,
                        void* dst, int accumulate);

/* SelectNode (ginn/node/select.h:24-112): dst[i] = cond[i] ? a : b, cond one
 * byte per element (Tensor<bool>); a branch flagged scalar is a single value
 * used for every i.  Backward: dst[i] += dy[i] where (cond[i] != 0) == want,
 * summed into dst[0] when the branch is a single value.  ginn_hip_select also
 * takes GINN_HIP_I32 (Select on Int, test/nodes.cu.cpp:825). */
int ginn_hip_select(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                    const unsigned char* cond, const void* a, int a_is_scalar,
                    const void* b, int b_is_scalar, void* dst);
int ginn_hip_select_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                        const unsigned char* cond, int want, const void* dy,
                        void* dst, int dst_is_scalar);

/* MaskNode (ginn/node/select.h:114-187): x viewed as [mask_size x batch];
 * dst (+)= mask != 0 ? x : value.  Forward with `value` = the mask value,
 * backward on the gradient with value 0 and accumulate.  dtype may be
 * GINN_HIP_I32 without accumulate (Mask on Int, test/nodes.cu.cpp:860): value
 * is then truncated to an integer. */
int ginn_hip_mask_select(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                         size_t mask_size, size_t batch, const void* mask,
                         float value, const void* x, void* dst, int accumulate);

/* LessThanNode (ginn/node/compare.h:27-56): out[i] = a[i] < b[i], one byte
 * each; dtype may be GINN_HIP_I32. */
int ginn_hip_less_than(ginn_hip_ctx* ctx, int dtype, size_t n, const void* a,
                       const void* b, unsigned char* out);

/* PickNode (ginn/node/pick.h:29-170): out[c] = x[idx[c], c] for a [rows x cols]
 * x (thrust::gather in the reference); backward dx[idx[c], c] += sign * dout[c]
 * (its gather + add + scatter).  An index outside [0, rows) picks NaN and
 * receives nothing. */
int ginn_hip_pick(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows, int cols,
                  const void* x, const int* idx, void* out);
int ginn_hip_pick_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                      int cols, const int* idx, const void* dout, float sign,
                      void* dx);

/* PickNegLogSigmoidNode (ginn/node/pick.h:250-304): sigm = sigmoid(x),
 * out = -(idx ? log sigm : log(1 - sigm)) elementwise, idx int32 of the same
 * shape; backward dx += (sigm - idx) * dout. */
int ginn_hip_pick_nlsig_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                            const void* x, const int* idx, void* sigm,
                            void* out);
int ginn_hip_pick_nlsig_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                            const void* sigm, const int* idx, const void* dout,
                            void* dx);

/* AxisSumNode (ginn/node/reduce.h:53-136): sums x over the axes flagged in
 * host_summed (HOST arrays of `rank` <= 8 entries); dst holds the remaining
 * axes in order.  Backward: dx[i] += dy[i projected onto the kept axes]. */
int ginn_hip_axis_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank,
                      const long long* host_dims, const int* host_summed,
                      const void* x, void* dst);
int ginn_hip_axis_sum_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rank,
                          const long long* host_dims, const int* host_summed,
                          const void* dy, void* dx);

/* VarianceNode (ginn/node/reduce.h:164-204): mean_out[0] = mean(x),
 * var_out[0] = mean((x - mean)^2); backward dx += (x - mean) * dvar * 2 / n. */
int ginn_hip_variance_fwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                          const void* x, void* mean_out, void* var_out);
int ginn_hip_variance_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                          const void* x, const void* mean, const void* dvar,
                          void* dx);

/* StackNode (ginn/node/layout.h:324-444): dst = the `count` arrays of `sz`
 * elements named by the DEVICE table dev_srcs, one after the other
 * (stack_helper); elements of 1, 2 or 4 bytes.  Backward: array k receives
 * src[k * sz ...] added atomically (stack_backward_helper; a table may name
 * an array several times); NULL entries are inputs without gradient. */
int ginn_hip_stack(ginn_hip_ctx* ctx, int elem_bytes, size_t sz, size_t count,
                   const void* const* dev_srcs, void* dst);
int ginn_hip_stack_bwd(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t sz,
                       size_t count, void* const* dev_dsts, const void* src);

/* argmax (ginn/util/amax.h:28-66) along the middle axis of x viewed as
 * [inner x len x outer]: out[inner x outer] int64 positions, the first
 * maximum wins. */
int ginn_hip_argmax(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t inner,
                    size_t len, size_t outer, const void* x, long long* out);

/* RowBroadcastNode (ginn/node/layout.h:831-862): dst[r, c] = x[c]; its
 * backward is the column sum dst[c] (+)= sum_r x[r, c]. */
int ginn_hip_row_broadcast(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                           int cols, const void* x, void* dst);
int ginn_hip_col_sum(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, int rows,
                     int cols, const void* x, void* dst, int accumulate);

/* ------------------------------------------------------------------ */
/* Many elementwise operations in one launch                            */
/* ------------------------------------------------------------------ */

typedef enum {
  GINN_HIP_MULTI_FILL = 0,       /* dst = value */
  GINN_HIP_MULTI_SUM = 1,        /* dst = src0 (+ src1 (+ src2)); with one source: a copy */
  GINN_HIP_MULTI_PROD = 2,       /* dst = src0 * src1 */
  GINN_HIP_MULTI_NONLIN_FWD = 3, /* dst = act(src0) */
  GINN_HIP_MULTI_NONLIN_BWD = 4  /* dst = act'(x = src1, y = src2) * src0 (dy) */
} ginn_hip_multi_kind;

/* What the reference does with one Eigen expression per node
 * (ginn/node/common.h:97-157, 233-262, ginn/node/nlnode.h, ginn/node/layout.h)
 * for `count` independent nodes of the same kind and size n at once: operation
 * i reads dev_src*[i] and writes (accumulate != 0: adds into) dev_dst[i].  The
 * tables are DEVICE arrays of `count` device pointers; unused source tables
 * are NULL.  Destinations of one call must not overlap.  act is used by the
 * NONLIN kinds (any elementwise activation, not SOFTMAX). */
int ginn_hip_multi_apply(ginn_hip_ctx* ctx, ginn_hip_dtype dtype,
                         ginn_hip_multi_kind kind, ginn_hip_act act,
                         int accumulate, float value, size_t n, int count,
                         void* const* dev_dst, const void* const* dev_src0,
                         const void* const* dev_src1,
                         const void* const* dev_src2);

/* The same for operations that differ in kind, length or scalar type: every
 * element-wise node of one height of a graph in one launch, whatever it
 * computes.  dev_ops is a DEVICE array of `count` records; max_n >= every n
 * sizes the launch.  The fields mean what the arguments of
 * ginn_hip_multi_apply mean (unused sources NULL; the records are not
 * validated: they are in device memory).  Destinations must not overlap. */
typedef struct ginn_hip_multi_op {
  int dtype;      /* ginn_hip_dtype */
  int kind;       /* ginn_hip_multi_kind */
  int act;        /* ginn_hip_act, NONLIN kinds */
  int accumulate; /* != 0: add into dst */
  float value;    /* FILL */
  int reserved;   /* 0 */
  size_t n;       /* elements */
  void* dst;
  const void* src[3];
} ginn_hip_multi_op;
int ginn_hip_multi_mixed(ginn_hip_ctx* ctx, int count,
                         const ginn_hip_multi_op* dev_ops, size_t max_n);

/* Operations that depend on each other, as chains: chain b is the records
 * [first, first + count) of dev_ops, run in this order by one workgroup; the
 * `reserved` field of a record is its stage, ascending along a chain: records
 * of one stage are independent, a record may read what records of earlier
 * stages of ITS chain wrote.  Different chains (`count` of them) must be independent (no record
 * of one writes what a record of another reads or writes).  One launch then
 * does the work of one ginn_hip_multi_mixed launch per stage; meant for many
 * chains of small operations (the element-wise nodes between two products
 * of a recurrent cell, one chain per sequence).  No counterpart in the
 * reference, which launches every node on its own. */
typedef struct ginn_hip_chain_range {
  unsigned first; /* index of the chain's first record in dev_ops */
  unsigned count; /* records */
} ginn_hip_chain_range;
int ginn_hip_multi_chain(ginn_hip_ctx* ctx, int count,
                         const ginn_hip_chain_range* dev_chains,
                         const ginn_hip_multi_op* dev_ops);

/* dst[i] = (accumulate ? dst[i] : 0) + sum over k < count of dev_srcs[k][i],
 * i < n: what `count` users of one node do one after the other when each adds
 * its gradient into the node's (`in->grad() += grad()`, e.g.
 * ginn/node/common.h:131-137), as one reduction.  dev_srcs is a DEVICE array
 * of device pointers.  The order of summation is fixed by the table. */
int ginn_hip_multi_reduce(ginn_hip_ctx* ctx, ginn_hip_dtype dtype, size_t n,
                          int count, const void* const* dev_srcs, void* dst,
                          int accumulate);

/* Zero-fills `count` regions in one launch: region i is dev_bytes[i] bytes at
 * dev_ptrs[i] (both DEVICE arrays); max_bytes >= every dev_bytes[i] sizes the
 * launch.  What Graph::reset_grad() does with one grad().set_zero() per node
 * (ginn/node.h:197-200, 261-264; ginn/tensor.h:443). */
int ginn_hip_multi_zero(ginn_hip_ctx* ctx, int count, void* const* dev_ptrs,
                        const size_t* dev_bytes, size_t max_bytes);

/* ------------------------------------------------------------------ */
/* Weight updates  (ginn/update/update.h:54-168)                       */
/* ------------------------------------------------------------------ */

typedef enum { GINN_HIP_UPDATE_SGD = 0, GINN_HIP_UPDATE_ADAM = 1 } ginn_hip_update_kind;

/* One update rule with its constants as the reference forms them
 * (ginn/update/update.h:69-72 Sgd, :115-133 Adam).  SGD uses lr and clip.
 * Adam uses clip, beta1, one_minus_beta1 = (float)(1. - beta1), beta2,
 * one_minus_beta2, step = (float)(-lr * (1. / (1. - beta1^t))),
 * vscale = (float)(1. / (1. - beta2^t)) and eps, t counting this step. */
typedef struct ginn_hip_update_rule {
  int kind; /* ginn_hip_update_kind */
  float lr;
  float clip;
  float beta1, one_minus_beta1;
  float beta2, one_minus_beta2;
  float step, vscale, eps;
} ginn_hip_update_rule;

/* One weight: n elements of `dtype` at w with gradient g; m and v are its
 * fp32 Adam histories (NULL for SGD). */
typedef struct ginn_hip_update_op {
  void* w;
  void* g;
  float* m;
  float* v;
  size_t n;
  int dtype; /* ginn_hip_dtype */
  int reserved;
} ginn_hip_update_op;

/* One step of the rule on one weight, in place: the gradient is clipped
 * element-wise to [-clip, clip] and stored back, then
 *   SGD:  w += (-lr) * g            (Sgd::update, ginn/update/update.h:69-72)
 *   Adam: m = beta1 m + (1 - beta1) g,  v = beta2 v + (1 - beta2) g^2,
 *         w += (step * m) / (eps + sqrt(vscale * v))   (Adam::update, :115-133)
 * Every operation is rounded on its own in fp32 (no fused multiply-add); a
 * 16-bit weight receives the increment rounded to its type, as the
 * reference's cast.  Replaces the four to eight Eigen expression kernels of
 * one update by one pass over the weight. */
int ginn_hip_update(ginn_hip_ctx* ctx, const ginn_hip_update_rule* rule,
                    ginn_hip_dtype dtype, size_t n, void* w, void* g, float* m,
                    float* v);

/* The same step for `count` weights in one launch (Updater::update(Graph&),
 * ginn/update/update.h:36-48, which visits the weights one by one).  dev_ops
 * is a DEVICE array of `count` records that the caller keeps; max_n >= every
 * n sizes the launch.  The weights must not overlap. */
int ginn_hip_multi_update(ginn_hip_ctx* ctx, const ginn_hip_update_rule* rule,
                          int count, const ginn_hip_update_op* dev_ops,
                          size_t max_n);

/* ------------------------------------------------------------------ */
/* Recording the launches of a context and replaying them              */
/* ------------------------------------------------------------------ */

/* No counterpart in the reference (it launches every kernel of every pass
 * from the host).  Between capture_begin and capture_end the calls of this
 * library on `ctx` are recorded instead of run (HIP stream capture; nothing
 * that waits for the device or copies to or from the host may be called);
 * capture_end returns the recording, graph_launch replays it on the
 * context's stream with the very same arguments: pointers, sizes and scalars
 * are frozen, the contents of the buffers are read anew at every replay. */
typedef struct ginn_hip_graph ginn_hip_graph;
int ginn_hip_capture_begin(ginn_hip_ctx* ctx);
int ginn_hip_capture_end(ginn_hip_ctx* ctx, ginn_hip_graph** graph);
int ginn_hip_graph_launch(ginn_hip_graph* graph);
/* Kernel launches in the recording (what one replay runs on the device). */
int ginn_hip_graph_kernel_count(ginn_hip_graph* graph, size_t* kernels);
int ginn_hip_graph_destroy(ginn_hip_graph* graph);

/* ------------------------------------------------------------------ */
/* Timing on the context's stream (the role of GINN_TIME,              */
/* ginn/util/timer.h:244-249, without the device-wide synchronisation) */
/* ------------------------------------------------------------------ */

/* Records event slot `slot` (0..63) on the stream. */
int ginn_hip_event_record(ginn_hip_ctx* ctx, int slot);
/* Waits for slot `stop` and returns the milliseconds since slot `start`. */
int ginn_hip_event_elapsed_ms(ginn_hip_ctx* ctx, int start, int stop,
                              float* ms);

/* Library version, "major.minor". */
const char* ginn_hip_version(void);

#ifdef __cplusplus
}
#endif

#endif /* GINN_HIP_H */
