// Picking one row per column (ginn/node/pick.h): Pick, PickSoftmax,
// PickNegLogSoftmax (the softmax + negative log-likelihood head) and the
// elementwise PickNegLogSigmoid.  The index is an Int data node with one entry
// per column, a vector of indices, or a single index.
#ifndef GINN_NODE_PICK_H
#define GINN_NODE_PICK_H

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

namespace internal {
inline DataPtr<Int> index_node(const DevPtr& dev, const std::vector<Int>& index) {
  auto node = Data<Int>(dev, Shape{static_cast<Size>(index.size())});
  node->value().set(index);
  return node;
}
}  // namespace internal

// value[0, c] = x[index[c], c]; backward dx[index[c], c] += dy[c]
// (ginn/node/pick.h:29-170).
template <typename Scalar>
class PickNode : public BaseDataNode<Scalar> {
 protected:
  NodePtr<Scalar> in_;
  DataPtr<Int> index_;

  void check_index(const Tensor<Scalar>& input) const {
    GINN_ASSERT(input.cols() == index_->value().size(),
                "Index size does not match input columns! (" + std::to_string(index_->value().size()) + " != " +
                    std::to_string(input.cols()) + ")");
    GINN_ASSERT(index_->dev()->kind() == GPU, "Pick: the index tensor must live on the GPU");
  }
  // value() = one entry per column of `input`.
  void pick(const Tensor<Scalar>& input) {
    internal::require_gpu(this->dev(), "Pick");
    check_index(input);
    value().resize(1, input.cols());
    GINN_HIP_CALL(ginn_hip_pick(internal::ctx_of(input), dtype_of<Scalar>(), static_cast<int>(input.rows()),
                                static_cast<int>(input.cols()), input.data(), index_->value().data(),
                                value().data()));
  }
  // grad_in[index[c], c] += (or -=) grad()[c].
  void pick_grad(Tensor<Scalar>& grad_in, bool negate = false) {
    GINN_HIP_CALL(ginn_hip_pick_bwd(internal::ctx_of(grad_in), dtype_of<Scalar>(), static_cast<int>(grad_in.rows()),
                                    static_cast<int>(grad_in.cols()), index_->value().data(), grad().data(),
                                    negate ? -1.f : 1.f, grad_in.data()));
  }
  void forward_() override { pick(in_->value()); }
  void backward_() override {
    if (in_->has_grad()) pick_grad(in_->grad());
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  PickNode(const NodePtr<Scalar>& in, const DataPtr<Int>& index)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{in, index}), in_(in), index_(index) {}
  PickNode(const NodePtr<Scalar>& in, const std::vector<Int>& index)
      : PickNode(in, internal::index_node(in->dev(), index)) {}
  PickNode(const NodePtr<Scalar>& in, Int index) : PickNode(in, std::vector<Int>{index}) {}
  std::string name() const override { return "Pick"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Pick);

// Pick from the column softmax of x (ginn/node/pick.h:171-201).
template <typename Scalar>
class PickSoftmaxNode : public PickNode<Scalar> {
 protected:
  using PickNode<Scalar>::in_;
  Tensor<Scalar> smax_;

  void forward_() override {
    smax_.move_to(this->dev());
    SoftmaxOp<Scalar>().forward(smax_, in_->value());
    this->pick(smax_);
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    Tensor<Scalar> dsmax(smax_.dev(), smax_.shape());
    dsmax.set_zero();
    this->pick_grad(dsmax);
    SoftmaxOp<Scalar>().backward(in_->grad(), dsmax, in_->value(), smax_, true);
  }

 public:
  using PickNode<Scalar>::PickNode;
  std::string name() const override { return "PickSoftmax"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(PickSoftmax);

// value[0, c] = -log softmax(x)[index[c], c]; backward dx += softmax * dy
// (broadcast down the column), dx[index[c], c] -= dy[c]
// (ginn/node/pick.h:203-248).  Forward and backward are one kernel each.  The
// reference keeps the softmax matrix for backward; here forward keeps the
// maximum and the sum of exponentials of every column (two floats) and backward
// rebuilds the softmax from the input, rounded as it would have been stored:
// the same gradient, and forward writes [1 x cols] instead of [rows x cols].
template <typename Scalar>
class PickNegLogSoftmaxNode : public PickSoftmaxNode<Scalar> {
  using PickSoftmaxNode<Scalar>::in_;
  using PickNode<Scalar>::index_;
  Tensor<float> stats_;  // per column: maximum, 1 / sum of exp(x - maximum)

  void forward_() override {
    auto& x = in_->value();
    if (this->dev()->kind() == CPU) {  // the host layer's loops (ginn/cpu_ops.h)
      GINN_ASSERT(x.cols() == index_->value().size(), "Index size does not match input columns!");
      GINN_ASSERT(index_->dev()->kind() == CPU, "PickNegLogSoftmax: index and input must live on one device");
      value().resize(1, x.cols());
      host::pick_nls_forward<Scalar>(static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(),
                                    index_->value().data(), value().data());
      return;
    }
    internal::require_gpu(this->dev(), "PickNegLogSoftmax");
    this->check_index(x);
    stats_.move_to(this->dev());
    stats_.resize(2, x.cols());
    value().resize(1, x.cols());
    GINN_HIP_CALL(ginn_hip_pick_nls_fwd_stats(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<int>(x.rows()),
                                              static_cast<int>(x.cols()), x.data(), index_->value().data(),
                                              stats_.data(), value().data()));
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    auto& x = in_->value();
    const bool fresh = in_->take_lazy_zero();
    if (this->dev()->kind() == CPU) {
      host::pick_nls_backward<Scalar>(static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(),
                                     index_->value().data(), grad().data(), in_->grad().data(), !fresh);
      return;
    }
    GINN_HIP_CALL(ginn_hip_pick_nls_bwd_stats(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<int>(x.rows()),
                                              static_cast<int>(x.cols()), x.data(), stats_.data(),
                                              index_->value().data(), grad().data(), in_->grad().data(),
                                              fresh ? 0 : 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  using PickSoftmaxNode<Scalar>::PickSoftmaxNode;
  BaseNode::GradUse grad_use(size_t index) const override {
    return index == 0 ? BaseNode::GradUse::Overwrites : BaseNode::GradUse::Accumulates;
  }
  std::string name() const override { return "PickNegLogSoftmax"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(PickNegLogSoftmax);

// Elementwise binary cross-entropy on logits: value = -(index ? log s : log(1 - s)),
// s = sigmoid(x), index an Int tensor of x's shape; backward dx += (s - index) * dy
// (ginn/node/pick.h:250-304).
template <typename Scalar>
class PickNegLogSigmoidNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  DataPtr<Int> index_;
  Tensor<Scalar> sigm_;

  void forward_() override {
    internal::require_gpu(this->dev(), "PickNegLogSigmoid");
    auto& x = in_->value();
    GINN_ASSERT(index_->value().size() == x.size(), "PickNegLogSigmoid: one index per element expected");
    GINN_ASSERT(index_->dev()->kind() == GPU, "PickNegLogSigmoid: the index tensor must live on the GPU");
    sigm_.move_to(this->dev());
    sigm_.resize(x.shape());
    value().resize(x.shape());
    GINN_HIP_CALL(ginn_hip_pick_nlsig_fwd(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<size_t>(x.size()),
                                          x.data(), index_->value().data(), sigm_.data(), value().data()));
  }
  void backward_() override {
    if (in_->has_grad())
      GINN_HIP_CALL(ginn_hip_pick_nlsig_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                            static_cast<size_t>(grad().size()), sigm_.data(), index_->value().data(),
                                            grad().data(), in_->grad().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  PickNegLogSigmoidNode(const NodePtr<Scalar>& in, const DataPtr<Int>& index)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{in, index}), in_(in), index_(index), sigm_(in->dev()) {}
  PickNegLogSigmoidNode(const NodePtr<Scalar>& in, const std::vector<Int>& index)
      : PickNegLogSigmoidNode(in, internal::index_node(in->dev(), index)) {}
  PickNegLogSigmoidNode(const NodePtr<Scalar>& in, Int index) : PickNegLogSigmoidNode(in, std::vector<Int>{index}) {}
  std::string name() const override { return "PickNegLogSigmoid"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(PickNegLogSigmoid);

}  // namespace ginn

#endif  // GINN_NODE_PICK_H
