// Unary nonlinearity nodes: Tanh(x), Sigmoid(x), ... (ginn/node/nlnode.h:24-80).
#ifndef GINN_NODE_NLNODE_H
#define GINN_NODE_NLNODE_H

#include <ginn/node/data.h>
#include <ginn/nonlin.h>

namespace ginn {

#define GINN_MAKE_UNARY_NODE_AND_FACTORY(F)                                    \
  template <typename Scalar>                                                   \
  class F##Node : public BaseDataNode<Scalar> {                                \
   protected:                                                                  \
    NodePtr<Scalar> in_;                                                       \
    F##Op<Scalar> op_{};                                                       \
    void forward_() override { op_.forward(value(), in_->value()); }           \
    void backward_() override {                                                \
      if (!in_->has_grad()) return;                                            \
      const bool fresh = in_->take_lazy_zero();                                \
      op_.backward(in_->grad(), grad(), in_->value(), value(), !fresh);        \
    }                                                                          \
                                                                               \
   public:                                                                     \
    using BaseDataNode<Scalar>::value;                                         \
    using BaseDataNode<Scalar>::grad;                                          \
    using UnaryOp = F##Op<Scalar>;                                             \
    BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; } \
    bool describe_forward(std::vector<LaunchDesc>& out) override {             \
      if (value().dev()->kind() != GPU || op_.code() == GINN_HIP_ACT_SOFTMAX) return false; \
      value().resize(in_->value().shape());                                    \
      LaunchDesc d;                                                            \
      d.dtype = dtype_of<Scalar>();                                            \
      d.kind = GINN_HIP_MULTI_NONLIN_FWD;                                      \
      d.act = op_.code();                                                      \
      d.n = static_cast<size_t>(value().size());                               \
      d.dst = value().data();                                                  \
      d.src[0] = in_->value().data();                                          \
      out.push_back(d);                                                        \
      return true;                                                             \
    }                                                                          \
    bool describe_backward(std::vector<LaunchDesc>& out) override {            \
      if (value().dev()->kind() != GPU || op_.code() == GINN_HIP_ACT_SOFTMAX) return false; \
      if (!in_->has_grad()) return true;                                       \
      LaunchDesc d;                                                            \
      d.dtype = dtype_of<Scalar>();                                            \
      d.kind = GINN_HIP_MULTI_NONLIN_BWD;                                      \
      d.act = op_.code();                                                      \
      d.accumulate = !in_->take_lazy_zero();                                   \
      d.n = static_cast<size_t>(value().size());                               \
      d.dst = in_->grad().data();                                              \
      d.src[0] = grad().data();                                                \
      d.src[1] = in_->value().data();                                          \
      d.src[2] = value().data();                                               \
      out.push_back(d);                                                        \
      return true;                                                             \
    }                                                                          \
    F##Node(const NodePtr<Scalar>& in) : BaseDataNode<Scalar>({in}), in_(in) {} \
    void set_ins(const std::vector<BaseNodePtr>& ins) override {               \
      GINN_ASSERT(ins.size() == 1);                                            \
      BaseNode::ins_ = ins;                                                    \
      in_ = dynamic_ptr_cast<Node<Scalar>>(ins.front());                       \
    }                                                                          \
    std::string name() const override { return #F; }                           \
  };                                                                           \
  GINN_MAKE_SCALAR_FORWARDING_FACTORY(F)

GINN_MAKE_UNARY_NODE_AND_FACTORY(Identity);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Tanh);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Sigmoid);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Relu);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Softmax);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Log);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Sqrt);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Gelu);
GINN_MAKE_UNARY_NODE_AND_FACTORY(Gelu2);

// The same node writing over its input: value() and grad() are the input's
// tensors, the backward pass rescales the gradient where it is instead of
// adding to it (ginn/node/nlnode.h:72-97).
#define GINN_MAKE_INPLACE_UNARY_NODE_AND_FACTORY(F)                            \
  template <typename Scalar>                                                   \
  class InPlace##F##Node : public F##Node<Scalar> {                            \
   protected:                                                                  \
    using F##Node<Scalar>::in_;                                                \
    using F##Node<Scalar>::op_;                                                \
    void backward_() override {                                                \
      if (in_->has_grad()) op_.backward(in_->grad(), in_->grad(), in_->value(), in_->value(), false); \
    }                                                                          \
                                                                               \
   public:                                                                     \
    const Tensor<Scalar>& value() const override { return std::as_const(*in_).value(); } \
    const Tensor<Scalar>& grad() const override { return std::as_const(*in_).grad(); }   \
    using Node<Scalar>::value;                                                 \
    using Node<Scalar>::grad;                                                  \
    bool has_grad() const override { return in_->has_grad(); }                 \
    GINN_GRAD_IS_ALIAS_OF(in_)                                                 \
    bool describe_forward(std::vector<LaunchDesc>&) override { return false; } \
    bool describe_backward(std::vector<LaunchDesc>&) override { return false; } \
    using UnaryOp = F##Op<Scalar>;                                             \
    using F##Node<Scalar>::F##Node;                                            \
    std::string name() const override { return "InPlace" #F; }                 \
  };                                                                           \
  GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlace##F)

GINN_MAKE_INPLACE_UNARY_NODE_AND_FACTORY(Sigmoid);

}  // namespace ginn

#endif  // GINN_NODE_NLNODE_H
