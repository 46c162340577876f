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

// Softmax down the columns.  Directly after InPlaceMask (and InPlaceProdScalar
// before that) whose work is still pending -- the score chain of an attention
// block, examples/min-gpt.cu.cpp:127-133 -- the three steps run as one launch,
// forward and, when the scores' gradient holds no value yet, backward; the
// results are those of the separate nodes, bit for bit.
template <typename Scalar>
using ColumnSoftmaxOp = SoftmaxOp<Scalar>;
GINN_MAKE_UNARY_NODE_AND_FACTORY(ColumnSoftmax);

template <typename Scalar>
class SoftmaxNode : public ColumnSoftmaxNode<Scalar> {
  using Base = ColumnSoftmaxNode<Scalar>;
  using Base::in_;

  struct Chain {
    PendingInPlace* mask_step = nullptr;
    PendingInPlace* scale_step = nullptr;  // may be absent
    Node<Scalar>* mask = nullptr;
    Node<Scalar>* scores = nullptr;  // the node whose storage the steps write over
  };
  // The in-place steps directly before this node, if they are a mask step with
  // an optional scale step below.
  Chain chain() const {
    Chain c;
    auto* m = dynamic_cast<PendingInPlace*>(in_.get());
    if (!m || m->pending_step() != PendingInPlace::Step::Mask) return c;
    auto* mask = dynamic_cast<Node<Scalar>*>(m->pending_mask());
    BaseNode* below = m->pending_input();
    auto* p = dynamic_cast<PendingInPlace*>(below);
    if (p && p->pending_step() == PendingInPlace::Step::Scale) {
      c.scale_step = p;
      below = p->pending_input();
    }
    auto* scores = dynamic_cast<Node<Scalar>*>(below);
    if (!mask || !scores) return Chain{};
    c.mask_step = m;
    c.mask = mask;
    c.scores = scores;
    return c;
  }

  void forward_() override {
    const Chain c = chain();
    // Pending below means: nobody has read the scaled / masked scores yet.  A
    // scale step that has run already (somebody read its value) counts as 1.
    if (!c.mask_step || !c.mask_step->pending() || in_->dev()->kind() != GPU) {
      Base::forward_();
      return;
    }
    float scale = 1.f;
    if (c.scale_step && c.scale_step->pending()) {
      scale = c.scale_step->pending_value();
      c.scale_step->take_pending();
    }
    c.mask_step->take_pending();
    Tensor<Scalar>& x = c.scores->value();
    this->value().resize(x.shape());
    GINN_HIP_CALL(ginn_hip_scaled_masked_softmax_fwd(
        internal::ctx_of(x), dtype_of<Scalar>(), static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(),
        scale, c.mask->value().data(), static_cast<size_t>(c.mask->value().size()), c.mask_step->pending_value(),
        this->value().data()));
  }

  void backward_() override {
    if (!in_->has_grad()) return;
    const Chain c = chain();
    // A flagged gradient below means: this node is the only user of the mask
    // step, that of the scale step, and so on down to the scores (BaseNode::GradUse).
    if (!c.mask_step || !in_->lazy_zero() || in_->dev()->kind() != GPU) {
      Base::backward_();
      return;
    }
    in_->take_lazy_zero();
    const Tensor<Scalar>& y = this->value();
    GINN_HIP_CALL(ginn_hip_scaled_masked_softmax_bwd(
        internal::ctx_of(y), dtype_of<Scalar>(), static_cast<int>(y.rows()), static_cast<int>(y.cols()),
        this->grad().data(), y.data(), c.scale_step ? c.scale_step->pending_value() : 1.f, c.mask->value().data(),
        static_cast<size_t>(c.mask->value().size()), in_->grad().data()));
    c.mask_step->skip_next_backward();
    if (c.scale_step) c.scale_step->skip_next_backward();
  }

 public:
  using Base::Base;
  using UnaryOp = SoftmaxOp<Scalar>;
  std::string name() const override { return "Softmax"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Softmax);
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
