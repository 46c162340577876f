// LayerNorm over dimension 0 (each column of the rank-2 fold is normalised),
// ginn/node/layernorm.h:25-92.  The per-column standard deviations are kept
// in fp32 whatever the scalar type; the backward pass is one fused kernel
// (the reference runs a degenerate batched product for the dy . y term).
#ifndef GINN_NODE_LAYERNORM_H
#define GINN_NODE_LAYERNORM_H

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

template <typename Scalar>
class CwiseProdAddNode;

// The normalisation is postponed until the value is read: a CwiseProdAdd right
// behind it (the gamma / beta step, examples/min-gpt.cu.cpp:100-103) then runs
// both as one pass (ginn_hip_layernorm_affine_fwd), and, when this node's
// gradient has no other user, both backward steps as one
// (ginn_hip_layernorm_affine_bwd).  Any other reader gets the value as usual.
template <typename Scalar>
class LayerNormNode : public BaseDataNode<Scalar>, public PostponedValue {
  friend class CwiseProdAddNode<Scalar>;

 protected:
  NodePtr<Scalar> in_;
  float eps_;
  Tensor<float> std_;
  mutable bool pending_ = false;  // forward() has run, the kernel has not
  bool skip_backward_ = false;    // the node behind has done this node's backward as well

  // Nodes that normalise in place run at once.
  virtual bool may_postpone() const { return true; }
  Tensor<Scalar>& raw_value() const { return const_cast<Tensor<Scalar>&>(BaseDataNode<Scalar>::value()); }
  void normalise() const {
    auto& x = in_->value();
    Tensor<Scalar>& y = may_postpone() ? raw_value() : const_cast<LayerNormNode*>(this)->value();
    if (x.dev()->kind() == CPU) {
      host::layernorm_forward<Scalar>(static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(), eps_, y.data(),
                                      const_cast<Tensor<float>&>(std_).data());
      return;
    }
    GINN_HIP_CALL(ginn_hip_layernorm_fwd(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<int>(x.rows()),
                                         static_cast<int>(x.cols()), x.data(), eps_, y.data(),
                                         const_cast<Tensor<float>&>(std_).data()));
  }
  void forward_() override {
    const Shape s = in_->shape();
    const Size rows = s.empty() ? 1 : s[0];
    std_.resize({1, rows > 0 ? Tensor<Scalar>::size(s) / rows : 0});
    if (may_postpone()) {
      raw_value().resize(s);
      pending_ = true;
    } else {
      value().resize(s);
      normalise();
    }
  }
  void backward_() override {
    if (skip_backward_) {
      skip_backward_ = false;
      return;
    }
    if (!in_->has_grad()) return;
    auto& y = value();
    const bool fresh = in_->take_lazy_zero();
    if (y.dev()->kind() == CPU) {
      host::layernorm_backward<Scalar>(static_cast<int>(y.rows()), static_cast<int>(y.cols()), grad().data(), y.data(),
                                       std_.data(), in_->grad().data(), !fresh);
      return;
    }
    GINN_HIP_CALL((fresh ? ginn_hip_layernorm_bwd_assign : ginn_hip_layernorm_bwd)(
        internal::ctx_of(y), dtype_of<Scalar>(), static_cast<int>(y.rows()), static_cast<int>(y.cols()),
        grad().data(), y.data(), std_.data(), in_->grad().data()));
  }

 public:
  const Tensor<Scalar>& value() const override {
    if (pending_) {
      pending_ = false;
      normalise();
    }
    return BaseDataNode<Scalar>::value();
  }
  using Node<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  void settle_value() override { (void)std::as_const(*this).value(); }
  Shape shape() const override { return pending_ ? in_->shape() : value().shape(); }
  DevPtr dev() const override { return in_->dev(); }
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }
  LayerNormNode(const NodePtr<Scalar>& in, double eps = 1e-8)
      : BaseDataNode<Scalar>({in}), in_(in), eps_(static_cast<float>(eps)), std_(in->dev()) {}
  std::string name() const override { return "LayerNorm"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(LayerNorm);

}  // namespace ginn

#endif  // GINN_NODE_LAYERNORM_H
