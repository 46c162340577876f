// Comparison nodes (ginn/node/compare.h:27-56): LessThan(a, b) is a bool
// tensor, carries no gradient; a < b on node handles builds it.
#ifndef GINN_NODE_COMPARE_H
#define GINN_NODE_COMPARE_H

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

template <typename InScalar>
class LessThanNode : public BaseDataNode<bool> {
  NodePtr<InScalar> l_, r_;

  void forward_() override {
    internal::require_gpu(this->dev(), "LessThan");
    GINN_ASSERT(l_->value().size() == r_->value().size(), "LessThan: operand sizes differ");
    value().resize(l_->value().shape());
    int dtype;
    if constexpr (std::is_same_v<InScalar, Int>) dtype = GINN_HIP_I32;
    else dtype = dtype_of<InScalar>();
    GINN_HIP_CALL(ginn_hip_less_than(internal::ctx_of(l_->value()), dtype, static_cast<size_t>(value().size()),
                                     l_->value().data(), r_->value().data(),
                                     reinterpret_cast<unsigned char*>(value().data())));
  }

 public:
  using BaseDataNode<bool>::value;
  bool has_grad() const override { return false; }
  LessThanNode(const NodePtr<InScalar>& l, const NodePtr<InScalar>& r)
      : BaseDataNode<bool>(std::vector<BaseNodePtr>{l, r}), l_(l), r_(r) {}
  std::string name() const override { return "LessThan"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(LessThan);

template <typename Left, typename Right>
auto operator<(const Ptr<Left>& a, const Ptr<Right>& b) {
  using Scalar = typename Left::Scalar;
  return LessThan(NodePtr<Scalar>(a), NodePtr<Scalar>(b));
}

}  // namespace ginn

#endif  // GINN_NODE_COMPARE_H
