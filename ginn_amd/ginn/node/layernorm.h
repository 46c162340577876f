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
class LayerNormNode : public BaseDataNode<Scalar> {
 protected:
  NodePtr<Scalar> in_;
  float eps_;
  Tensor<float> std_;

  void forward_() override {
    internal::require_gpu(this->dev(), "LayerNorm");
    auto& x = in_->value();
    value().resize(x.shape());
    std_.resize({1, x.cols()});
    GINN_HIP_CALL(ginn_hip_layernorm_fwd(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<int>(x.rows()),
                                         static_cast<int>(x.cols()), x.data(), eps_, value().data(), std_.data()));
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    auto& y = value();
    const bool fresh = in_->take_lazy_zero();
    GINN_HIP_CALL((fresh ? ginn_hip_layernorm_bwd_assign : ginn_hip_layernorm_bwd)(
        internal::ctx_of(y), dtype_of<Scalar>(), static_cast<int>(y.rows()), static_cast<int>(y.cols()),
        grad().data(), y.data(), std_.data(), in_->grad().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }
  LayerNormNode(const NodePtr<Scalar>& in, double eps = 1e-8)
      : BaseDataNode<Scalar>({in}), in_(in), eps_(static_cast<float>(eps)), std_(in->dev()) {}
  std::string name() const override { return "LayerNorm"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(LayerNorm);

}  // namespace ginn

#endif  // GINN_NODE_LAYERNORM_H
