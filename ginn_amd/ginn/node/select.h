// Element selection (ginn/node/select.h): Select(if, then, else) over a bool
// tensor, and Mask(x, mask, value), which replaces the entries whose mask
// entry is 0 and lets the mask broadcast over trailing dimensions.
#ifndef GINN_NODE_SELECT_H
#define GINN_NODE_SELECT_H

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

// value[i] = if[i] ? then[i] : else[i]; a branch of shape {} is one value used
// everywhere, and its gradient is the sum over the selected entries
// (ginn/node/select.h:24-112).  On Int the forward pass alone (integers carry
// no gradient here).
template <typename Scalar>
class SelectNode : public BaseDataNode<Scalar> {
  NodePtr<bool> if_;
  NodePtr<Scalar> then_, else_;

  static bool is_scalar(const NodePtr<Scalar>& n) { return n->shape().empty(); }
  const unsigned char* cond() const { return reinterpret_cast<const unsigned char*>(if_->value().data()); }

  void forward_() override {
    internal::require_gpu(this->dev(), "Select");
    GINN_ASSERT(is_scalar(then_) || then_->shape() == if_->shape());
    GINN_ASSERT(is_scalar(else_) || else_->shape() == if_->shape());
    value().resize(if_->shape());
    GINN_HIP_CALL(ginn_hip_select(internal::ctx_of(value()), arith_dtype_of<Scalar>(), static_cast<size_t>(value().size()),
                                  cond(), then_->value().data(), is_scalar(then_) ? 1 : 0, else_->value().data(),
                                  is_scalar(else_) ? 1 : 0, value().data()));
  }
  void backward_() override {
    if constexpr (is_floating_point_v<Scalar>) {
      const size_t n = static_cast<size_t>(grad().size());
      if (then_->has_grad())
        GINN_HIP_CALL(ginn_hip_select_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(), n, cond(), 1, grad().data(),
                                          then_->grad().data(), is_scalar(then_) ? 1 : 0));
      if (else_->has_grad())
        GINN_HIP_CALL(ginn_hip_select_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(), n, cond(), 0, grad().data(),
                                          else_->grad().data(), is_scalar(else_) ? 1 : 0));
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  SelectNode(const NodePtr<bool>& if_n, const NodePtr<Scalar>& then_n, const NodePtr<Scalar>& else_n)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{if_n, then_n, else_n}), if_(if_n), then_(then_n), else_(else_n) {}
  SelectNode(const NodePtr<bool>& if_n, const NodePtr<Scalar>& then_n, Scalar else_val)
      : SelectNode(if_n, then_n, NodePtr<Scalar>(Constant<Scalar>(if_n->dev(), Shape{}, else_val))) {}
  SelectNode(const NodePtr<bool>& if_n, Scalar then_val, const NodePtr<Scalar>& else_n)
      : SelectNode(if_n, NodePtr<Scalar>(Constant<Scalar>(if_n->dev(), Shape{}, then_val)), else_n) {}
  SelectNode(const NodePtr<bool>& if_n, Scalar then_val, Scalar else_val)
      : SelectNode(if_n, NodePtr<Scalar>(Constant<Scalar>(if_n->dev(), Shape{}, then_val)),
                   NodePtr<Scalar>(Constant<Scalar>(if_n->dev(), Shape{}, else_val))) {}
  std::string name() const override { return "Select"; }
};

namespace internal {
template <typename X>
struct select_scalar {
  using type = std::decay_t<X>;
};
template <typename N>
struct select_scalar<Ptr<N>> {
  using type = typename N::Scalar;
};
template <typename Scalar, typename X>
decltype(auto) select_arg(X&& x) {
  if constexpr (is_node_ptr_v<X>) return NodePtr<Scalar>(x);
  else return Scalar(x);
}
}  // namespace internal

// Select(if, then, else): either branch may be a node or a plain value; the
// scalar type is that of the first branch (ginn/node/select.h:100-112).
template <typename If, typename Then, typename Else>
auto Select(const Ptr<If>& if_, Then&& then_, Else&& else_) {
  using Scalar = typename internal::select_scalar<std::decay_t<Then>>::type;
  return make_ptr<SelectNode<Scalar>>(NodePtr<bool>(if_), internal::select_arg<Scalar>(std::forward<Then>(then_)),
                                      internal::select_arg<Scalar>(std::forward<Else>(else_)));
}

// value = mask != 0 ? x : mask_val, the mask broadcast over the trailing
// dimensions in which it has extent 1; backward passes the gradient where the
// mask is set (ginn/node/select.h:114-187).
template <typename Scalar>
class MaskNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_, mask_;
  float mask_val_;

  void run(const Tensor<Scalar>& x, float val, Tensor<Scalar>& dst, bool accumulate) {
    const Size ms = mask_->value().size();
    GINN_HIP_CALL(ginn_hip_mask_select(internal::ctx_of(dst), arith_dtype_of<Scalar>(), static_cast<size_t>(ms),
                                       static_cast<size_t>(x.size() / ms), mask_->value().data(), val, x.data(),
                                       dst.data(), accumulate ? 1 : 0));
  }
  void forward_() override {
    internal::require_gpu(this->dev(), "Mask");
    const Shape ms = mask_->shape(), is = in_->shape();
    GINN_ASSERT(ms.size() == is.size());
    size_t i = 0;
    while (i < is.size() && ms[i] == is[i]) ++i;
    for (; i < is.size(); ++i) GINN_ASSERT(ms[i] == 1, "Unexpected mask shape!");
    GINN_ASSERT(mask_->value().size() > 0);
    value().resize(is);
    run(in_->value(), mask_val_, value(), false);
  }
  void backward_() override {
    if constexpr (is_floating_point_v<Scalar>)
      if (in_->has_grad()) run(grad(), 0.f, in_->grad(), true);
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  template <typename Val>
  MaskNode(const NodePtr<Scalar>& in, const NodePtr<Scalar>& mask, Val mask_val)
      : BaseDataNode<Scalar>({in, mask}), in_(in), mask_(mask),
        mask_val_(static_cast<float>(Scalar(static_cast<float>(mask_val)))) {}
  std::string name() const override { return "Mask"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Mask);

}  // namespace ginn

#endif  // GINN_NODE_SELECT_H
