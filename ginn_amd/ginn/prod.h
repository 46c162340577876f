// Device matrix-product routines of the host layer.
//
// Same entry points, argument order and shape checks as ginn/prod.h:32-310;
// the BLAS handle parameter becomes the libginn_hip.so context and the two
// cuBLAS calls become ginn_hip_gemm / ginn_hip_gemm_strided_batched.
#ifndef GINN_PROD_H
#define GINN_PROD_H

#include <ginn/cpu_ops.h>
#include <ginn/tensor.h>

namespace ginn {
namespace internal {

// Operation flags in the role of cublasOperation_t.
using GemmOp = ginn_hip_op;
constexpr GemmOp OP_N = GINN_HIP_OP_N;
constexpr GemmOp OP_T = GINN_HIP_OP_T;

// C[m x n] = op1(A)[m x k] * op2(B)[k x n] + bet * C.  Note the reference's
// argument order m, k, n (ginn/prod.h:32-45).
template <typename Scalar>
inline void gpu_gemm(ginn_hip_ctx*& handle, const Scalar* A, const Scalar* B, Scalar* C, const int lda,
                     const int ldb, const int ldc, const int m, const int k, const int n,
                     const Scalar bet = Scalar(0), const GemmOp& op1 = OP_N, const GemmOp& op2 = OP_N) {
  if constexpr (is_floating_point_v<Scalar>) {
    GINN_HIP_CALL(ginn_hip_gemm(handle, dtype_of<Scalar>(), op1, op2, m, n, k, A, lda, B, ldb,
                                static_cast<float>(bet), C, ldc));
  } else {
    GINN_THROW("Unexpected Scalar type in gpu_gemm!");
  }
}

// Strided-batched form (ginn/prod.h:68-135): operand i at base + i * stride.
template <typename Scalar>
inline void gpu_batched_gemm(ginn_hip_ctx*& handle, const Scalar* A, const Scalar* B, Scalar* C, const int lda,
                             const int ldb, const int ldc, const int sA, const int sB, const int sC,
                             const int m, const int k, const int n, const int batches,
                             const Scalar bet = Scalar(0), const GemmOp& op1 = OP_N, const GemmOp& op2 = OP_N) {
  if constexpr (is_floating_point_v<Scalar>) {
    GINN_HIP_CALL(ginn_hip_gemm_strided_batched(handle, dtype_of<Scalar>(), op1, op2, m, n, k, A, lda, sA, B,
                                                ldb, sB, static_cast<float>(bet), C, ldc, sC, batches));
  } else {
    GINN_THROW("Unexpected Scalar type in gpu_batched_gemm!");
  }
}

enum class ProdResult { Assign, Add };
enum class ProdTranspose { None, First, Second, Both };

// c (+)= op(a) * op(b) on the rank-2 folds of the tensors (ginn/prod.h:211-253).
// The first form runs on the context given (internal::BesidePass), the second on the context of c's GPU.
template <typename Scalar>
inline void gpu_prod(ginn_hip_ctx*& handle, Tensor<Scalar>& c, Tensor<Scalar>& a, Tensor<Scalar>& b,
                     ProdResult res = ProdResult::Assign, ProdTranspose tra = ProdTranspose::None) {
  const bool ta = tra == ProdTranspose::First || tra == ProdTranspose::Both;
  const bool tb = tra == ProdTranspose::Second || tra == ProdTranspose::Both;
  const Size a_outer = ta ? a.cols() : a.rows(), a_inner = ta ? a.rows() : a.cols();
  const Size b_outer = tb ? b.rows() : b.cols(), b_inner = tb ? b.cols() : b.rows();

  GINN_ASSERT(a_inner == b_inner);
  GINN_ASSERT(a_outer == c.rows());
  GINN_ASSERT(b_outer == c.cols());

  gpu_gemm<Scalar>(handle, a.data(), b.data(), c.data(),
                   /* lda */ static_cast<int>(a.rows()), /* ldb */ static_cast<int>(b.rows()),
                   /* ldc */ static_cast<int>(c.rows()), /* m */ static_cast<int>(a_outer),
                   /* k */ static_cast<int>(a_inner), /* n */ static_cast<int>(b_outer),
                   res == ProdResult::Add ? Scalar(1.f) : Scalar(0.f), ta ? OP_T : OP_N, tb ? OP_T : OP_N);
}
template <typename Scalar>
inline void gpu_prod(Tensor<Scalar>& c, Tensor<Scalar>& a, Tensor<Scalar>& b,
                     ProdResult res = ProdResult::Assign, ProdTranspose tra = ProdTranspose::None) {
  gpu_prod(cublas_handle(static_cast<int>(c.dev()->id().idx)), c, a, b, res, tra);
}

// c[:, :, i] (+)= op(a[:, :, i]) * op(b[:, :, i]) on the rank-3 folds
// (ginn/prod.h:256-310); strides are the full slice sizes.
template <typename Scalar>
inline void gpu_batched_prod(Tensor<Scalar>& c, Tensor<Scalar>& a, Tensor<Scalar>& b,
                             ProdResult res = ProdResult::Assign, ProdTranspose tra = ProdTranspose::None) {
  const Shape as = Tensor<Scalar>::reduce(a.shape(), 3), bs = Tensor<Scalar>::reduce(b.shape(), 3),
              cs = Tensor<Scalar>::reduce(c.shape(), 3);
  const Size a_rows = as[0], a_cols = as[1], batches = as[2];
  const Size b_rows = bs[0], b_cols = bs[1];
  const Size c_rows = cs[0], c_cols = cs[1];
  const bool ta = tra == ProdTranspose::First || tra == ProdTranspose::Both;
  const bool tb = tra == ProdTranspose::Second || tra == ProdTranspose::Both;
  const Size a_outer = ta ? a_cols : a_rows, a_inner = ta ? a_rows : a_cols;
  const Size b_outer = tb ? b_rows : b_cols, b_inner = tb ? b_cols : b_rows;

  GINN_ASSERT(a_inner == b_inner);
  GINN_ASSERT(a_outer == c_rows);
  GINN_ASSERT(b_outer == c_cols);

  gpu_batched_gemm<Scalar>(cublas_handle(static_cast<int>(c.dev()->id().idx)), a.data(), b.data(), c.data(),
                           static_cast<int>(a_rows), static_cast<int>(b_rows), static_cast<int>(c_rows),
                           static_cast<int>(a_rows * a_cols), static_cast<int>(b_rows * b_cols),
                           static_cast<int>(a_outer * b_outer), static_cast<int>(a_outer),
                           static_cast<int>(a_inner), static_cast<int>(b_outer), static_cast<int>(batches),
                           res == ProdResult::Add ? Scalar(1.f) : Scalar(0.f), ta ? OP_T : OP_N,
                           tb ? OP_T : OP_N);
}

// The same two products for tensors on cpu(): the host layer's own loops (ginn/cpu_ops.h), where the
// reference contracts with Eigen (ginn/node/prod.h:31-34,46-51).
template <typename Scalar>
inline void cpu_prod(Tensor<Scalar>& c, Tensor<Scalar>& a, Tensor<Scalar>& b, ProdResult res = ProdResult::Assign,
                     ProdTranspose tra = ProdTranspose::None) {
  const bool ta = tra == ProdTranspose::First || tra == ProdTranspose::Both;
  const bool tb = tra == ProdTranspose::Second || tra == ProdTranspose::Both;
  const Size a_outer = ta ? a.cols() : a.rows(), a_inner = ta ? a.rows() : a.cols();
  const Size b_outer = tb ? b.rows() : b.cols(), b_inner = tb ? b.cols() : b.rows();
  GINN_ASSERT(a_inner == b_inner);
  GINN_ASSERT(a_outer == c.rows());
  GINN_ASSERT(b_outer == c.cols());
  if constexpr (is_floating_point_v<Scalar>) {
    host::gemm<Scalar>(ta, tb, static_cast<int>(a_outer), static_cast<int>(b_outer), static_cast<int>(a_inner), a.data(),
                      static_cast<int>(a.rows()), b.data(), static_cast<int>(b.rows()),
                      res == ProdResult::Add ? 1.f : 0.f, c.data(), static_cast<int>(c.rows()));
  } else {
    GINN_THROW("Unexpected Scalar type in cpu_prod!");
  }
}
template <typename Scalar>
inline void cpu_batched_prod(Tensor<Scalar>& c, Tensor<Scalar>& a, Tensor<Scalar>& b,
                             ProdResult res = ProdResult::Assign, ProdTranspose tra = ProdTranspose::None) {
  const Shape as = Tensor<Scalar>::reduce(a.shape(), 3), bs = Tensor<Scalar>::reduce(b.shape(), 3),
              cs = Tensor<Scalar>::reduce(c.shape(), 3);
  const bool ta = tra == ProdTranspose::First || tra == ProdTranspose::Both;
  const bool tb = tra == ProdTranspose::Second || tra == ProdTranspose::Both;
  const Size a_outer = ta ? as[1] : as[0], a_inner = ta ? as[0] : as[1];
  const Size b_outer = tb ? bs[0] : bs[1], b_inner = tb ? bs[1] : bs[0];
  GINN_ASSERT(a_inner == b_inner);
  GINN_ASSERT(a_outer == cs[0]);
  GINN_ASSERT(b_outer == cs[1]);
  if constexpr (is_floating_point_v<Scalar>) {
    for (Size i = 0; i < as[2]; ++i)
      host::gemm<Scalar>(ta, tb, static_cast<int>(a_outer), static_cast<int>(b_outer), static_cast<int>(a_inner),
                        a.data() + i * as[0] * as[1], static_cast<int>(as[0]), b.data() + i * bs[0] * bs[1],
                        static_cast<int>(bs[0]), res == ProdResult::Add ? 1.f : 0.f, c.data() + i * cs[0] * cs[1],
                        static_cast<int>(cs[0]));
  } else {
    GINN_THROW("Unexpected Scalar type in cpu_batched_prod!");
  }
}

}  // namespace internal
}  // namespace ginn

#endif  // GINN_PROD_H
