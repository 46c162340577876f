// Reductions (ginn/node/reduce.h): Sum, Mean and Variance produce a rank-0
// tensor and broadcast the scalar gradient back; AxisSum sums over chosen axes.
#ifndef GINN_NODE_REDUCE_H
#define GINN_NODE_REDUCE_H

#include <algorithm>

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

template <typename Scalar>
class SumNode : public BaseDataNode<Scalar> {
 protected:
  NodePtr<Scalar> in_;
  virtual float scale() const { return 1.f; }

  void forward_() override {
    value().resize({});
    if (this->dev()->kind() == CPU) {
      value().data()[0] = Scalar(scale() * host::sum_all<Scalar>(static_cast<size_t>(in_->value().size()),
                                                                 in_->value().data()));
      return;
    }
    internal::require_gpu(this->dev(), name().c_str());
    GINN_HIP_CALL(ginn_hip_sum_all(internal::ctx_of(value()), dtype_of<Scalar>(),
                                   static_cast<size_t>(in_->value().size()), in_->value().data(), scale(),
                                   value().data()));
  }
  void backward_() override {
    if (in_->has_grad() && this->dev()->kind() == CPU) {
      const float g = scale() * static_cast<float>(grad().data()[0]);
      Scalar* dx = in_->grad().data();
      for (Size i = 0; i < in_->grad().size(); ++i) dx[i] = Scalar(static_cast<float>(dx[i]) + g);
      return;
    }
    if (in_->has_grad())
      GINN_HIP_CALL(ginn_hip_add_scalar_bcast(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                              static_cast<size_t>(in_->grad().size()), grad().data(), scale(),
                                              in_->grad().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  SumNode(const NodePtr<Scalar>& in) : BaseDataNode<Scalar>(in->dev(), Shape{}, {in}), in_(in) {}
  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() == 1);
    BaseNode::ins_ = ins;
    in_ = dynamic_ptr_cast<Node<Scalar>>(ins.front());
  }
  std::string name() const override { return "Sum"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Sum);

template <typename Scalar>
class MeanNode : public SumNode<Scalar> {
  float scale() const override { return 1.f / static_cast<float>(this->in_->value().size()); }

 public:
  using SumNode<Scalar>::SumNode;
  std::string name() const override { return "Mean"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Mean);

// Sum over the given axes (sorted, unique); the result keeps the other axes in
// order; backward broadcasts the gradient along the summed axes
// (ginn/node/reduce.h:53-136).
template <typename Scalar>
class AxisSumNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  std::vector<Size> axes_;
  std::vector<long long> dims_;
  std::vector<int> summed_;

  void forward_() override {
    internal::require_gpu(this->dev(), "AxisSum");
    const Shape in_s = in_->shape();
    GINN_ASSERT(!in_s.empty() && in_s.size() <= 8, "AxisSum: input rank must be 1..8");
    dims_.assign(in_s.begin(), in_s.end());
    summed_.assign(in_s.size(), 0);
    for (Size a : axes_) {
      GINN_ASSERT(a >= 0 && a < static_cast<Size>(in_s.size()), "AxisSum: axis out of range");
      summed_[static_cast<size_t>(a)] = 1;
    }
    Shape s;
    for (size_t j = 0; j < in_s.size(); ++j)
      if (!summed_[j]) s.push_back(in_s[j]);
    value().resize(s);
    GINN_HIP_CALL(ginn_hip_axis_sum(internal::ctx_of(value()), dtype_of<Scalar>(), static_cast<int>(dims_.size()),
                                    dims_.data(), summed_.data(), in_->value().data(), value().data()));
  }
  void backward_() override {
    if (in_->has_grad())
      GINN_HIP_CALL(ginn_hip_axis_sum_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                          static_cast<int>(dims_.size()), dims_.data(), summed_.data(), grad().data(),
                                          in_->grad().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  AxisSumNode(const NodePtr<Scalar>& in, std::vector<Size> axes)
      : BaseDataNode<Scalar>({in}), in_(in), axes_(std::move(axes)) {
    GINN_ASSERT(std::is_sorted(axes_.begin(), axes_.end()), "Axes need to be specified in sorted order in AxisSum!");
    GINN_ASSERT(std::adjacent_find(axes_.begin(), axes_.end()) == axes_.end(),
                "Axes need to be uniquely specified in AxisSum!");
  }
  std::string name() const override { return "AxisSum"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(AxisSum);

template <typename NodePtrType>
auto AxisSum(NodePtrType in, std::initializer_list<Size> axes) {
  return AxisSum(in, std::vector<Size>(axes));
}

// Biased variance of all elements; backward dx += (x - mean) * dy * 2 / n
// (ginn/node/reduce.h:164-204).
template <typename Scalar>
class VarianceNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Tensor<Scalar> mean_;

  void forward_() override {
    internal::require_gpu(this->dev(), "Variance");
    value().resize({});
    mean_.resize({});
    GINN_HIP_CALL(ginn_hip_variance_fwd(internal::ctx_of(value()), dtype_of<Scalar>(),
                                        static_cast<size_t>(in_->value().size()), in_->value().data(), mean_.data(),
                                        value().data()));
  }
  void backward_() override {
    if (in_->has_grad())
      GINN_HIP_CALL(ginn_hip_variance_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                          static_cast<size_t>(in_->value().size()), in_->value().data(), mean_.data(),
                                          grad().data(), in_->grad().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  VarianceNode(const NodePtr<Scalar>& in)
      : BaseDataNode<Scalar>(in->dev(), Shape{}, {in}), in_(in), mean_(in->dev(), Shape{}) {}
  std::string name() const override { return "Variance"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Variance);

}  // namespace ginn

#endif  // GINN_NODE_REDUCE_H
