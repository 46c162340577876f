// How the [rows x cols] slices of a batched product lie in memory when they are
// not a contiguous rank-3 tensor: a permutation of the axes of a rank-3 / rank-4
// tensor that keeps the first axis first (or second) only changes the leading
// dimension and the batch strides of its slices (or transposes them).  With
// that, BatchedProd reads the heads of an attention layer where the projections
// wrote them ([head size x heads x batch x time] after Reshape) and writes its
// result where the next projection reads it, and the Permute nodes between them
// (examples/min-gpt.cu.cpp:117-135; ginn/node/layout.h:723-821) copy nothing:
// a Permute postpones its copy until somebody reads its value, a BatchedProd
// behind or in front of it asks for the slices instead.
#ifndef GINN_NODE_SLICES_H
#define GINN_NODE_SLICES_H

#include <ginn/tensor.h>

namespace ginn {
namespace internal {

// Slice (z0, z1), z0 < n0, z1 < n1, is the column-major matrix with leading dimension ld at
// data + z0 * s0 + z1 * s1: [rows x cols], or with `transposed` the stored [cols x rows] transpose of it.
template <typename Scalar>
struct BatchView {
  Scalar* data = nullptr;
  Size rows = 0, cols = 0;
  Size ld = 0;
  long long s0 = 0, s1 = 0;
  Size n0 = 1, n1 = 1;
  bool transposed = false;
};

// The slices of a contiguous tensor of rank >= 3 (batch axes beyond the fourth fold into the third).
template <typename Scalar>
BatchView<Scalar> contiguous_slices(Tensor<Scalar>& t) {
  const Shape s = t.shape();
  BatchView<Scalar> v;
  v.data = t.data();
  v.rows = s[0];
  v.cols = s[1];
  v.ld = s[0];
  v.s0 = static_cast<long long>(s[0]) * s[1];
  if (s.size() == 4) {
    v.n0 = s[2];
    v.n1 = s[3];
  } else {
    v.n0 = 1;
    for (size_t i = 2; i < s.size(); ++i) v.n0 *= s[i];
    v.n1 = 1;
  }
  v.s1 = v.s0 * v.n0;
  return v;
}

// A tensor `viewed` with viewed[i_0, i_1, ...] = stored[...], where axis j of `viewed` runs along axis
// perm[j] of `stored` (PermuteNode: viewed = result, stored = input, perm = its indices): the slices
// viewed[:, :, z0, z1] inside the memory of `stored`.  False when they are no matrices there (neither of
// the first two axes of `viewed` is the contiguous axis of `stored`) or the rank is not 3 or 4.
template <typename Scalar>
bool permuted_slices(Scalar* stored, const Shape& stored_shape, const Shape& perm, BatchView<Scalar>& v) {
  const size_t rank = stored_shape.size();
  if ((rank != 3 && rank != 4) || perm.size() != rank) return false;
  long long stride[4];
  long long run = 1;
  for (size_t i = 0; i < rank; ++i) {
    stride[i] = run;
    run *= stored_shape[i];
  }
  auto axis = [&](size_t j) { return static_cast<size_t>(perm[j]); };
  if (axis(0) == 0) {
    v.transposed = false;
    v.ld = static_cast<Size>(stride[axis(1)]);
  } else if (axis(1) == 0) {
    v.transposed = true;
    v.ld = static_cast<Size>(stride[axis(0)]);
  } else {
    return false;
  }
  v.data = stored;
  v.rows = stored_shape[axis(0)];
  v.cols = stored_shape[axis(1)];
  v.s0 = stride[axis(2)];
  v.n0 = stored_shape[axis(2)];
  v.s1 = rank == 4 ? stride[axis(3)] : 0;
  v.n1 = rank == 4 ? stored_shape[axis(3)] : 1;
  return true;
}

// C = op(A) op(B) (+ C) slice by slice; ta / tb transpose the slices as their views describe them.
template <typename Scalar>
void batched_product(ginn_hip_ctx* ctx, BatchView<Scalar> C, BatchView<Scalar> A, bool ta, BatchView<Scalar> B, bool tb,
                     bool accumulate) {
  const Size am = ta ? A.cols : A.rows, ak = ta ? A.rows : A.cols;
  const Size bk = tb ? B.cols : B.rows, bn = tb ? B.rows : B.cols;
  GINN_ASSERT(ak == bk);
  GINN_ASSERT(am == C.rows);
  GINN_ASSERT(bn == C.cols);
  GINN_ASSERT(A.n0 * A.n1 == C.n0 * C.n1 && B.n0 * B.n1 == C.n0 * C.n1);
  // One numbering of the slices for all three: an operand that is contiguous follows the others.
  auto renumber = [](BatchView<Scalar>& v, Size n0, Size n1) {
    if (v.n0 == n0 && v.n1 == n1) return true;
    if (v.s1 != v.s0 * v.n0 && v.n1 != 1) return false;  // its two levels are not one run of slices
    v.n0 = n0;
    v.n1 = n1;
    v.s1 = v.s0 * n0;
    return true;
  };
  Size n0 = C.n0, n1 = C.n1;
  for (const BatchView<Scalar>* v : {&A, &B, &C})
    if (v->n1 != 1 && v->s1 != v->s0 * v->n0) {
      n0 = v->n0;
      n1 = v->n1;
    }
  GINN_ASSERT(renumber(A, n0, n1) && renumber(B, n0, n1) && renumber(C, n0, n1),
              "BatchedProd: the slices of the operands are numbered differently");
  bool sa = ta != A.transposed, sb = tb != B.transposed;  // relative to the stored matrices
  Size m = C.rows, n = C.cols;
  if (C.transposed) {  // the stored result is op(B)^T op(A)^T
    std::swap(A, B);
    const bool t = sa;
    sa = !sb;
    sb = !t;
    std::swap(m, n);
  }
  if constexpr (is_floating_point_v<Scalar>) {
    GINN_HIP_CALL(ginn_hip_gemm_strided_batched2(
        ctx, dtype_of<Scalar>(), sa ? GINN_HIP_OP_T : GINN_HIP_OP_N, sb ? GINN_HIP_OP_T : GINN_HIP_OP_N,
        static_cast<int>(m), static_cast<int>(n), static_cast<int>(ak), A.data, static_cast<int>(A.ld), A.s0, A.s1,
        B.data, static_cast<int>(B.ld), B.s0, B.s1, accumulate ? 1.f : 0.f, C.data, static_cast<int>(C.ld), C.s0, C.s1,
        static_cast<int>(n0), static_cast<int>(n1)));
  } else {
    GINN_THROW("Unexpected Scalar type in batched_product!");
  }
}

// A node whose value is a permutation of its input's that has not been carried out: hands out the slices
// of its value (and takes those of its gradient) inside its input's memory.
template <typename Scalar>
class SliceProvider {
 public:
  virtual ~SliceProvider() = default;
  // The slices of the value, if the copy is still pending; the copy then stays pending.
  virtual bool value_slices(BatchView<Scalar>& v) = 0;
  // From the node's only user, in the backward pass: where to put (accumulate: add) what it would have
  // written into the node's gradient -- the slices of the input's gradient.  The node then skips its own step.
  virtual bool grad_slices(BatchView<Scalar>& v, bool& accumulate) = 0;
};

// A node whose value is a batched product that has not been carried out.
template <typename Scalar>
class SliceTaker {
 public:
  virtual ~SliceTaker() = default;
  virtual bool product_pending() const = 0;
  // Carries the product out with its result written as the slices v (of a Permute node's value).
  virtual void produce_into(const BatchView<Scalar>& v) = 0;
  // From the node's only user, in the backward pass: the gradient of the node lies in the slices v.
  virtual bool take_grad_slices(const BatchView<Scalar>& v) = 0;
};

}  // namespace internal
}  // namespace ginn

#endif  // GINN_NODE_SLICES_H
