// Nodes that overwrite their input's storage: value() and grad() alias the
// input's tensors (ginn/node/inplace.h).  They save memory where the input
// value is not needed again; none of them is described to the level executor
// (they run themselves, in graph order).
#ifndef GINN_NODE_INPLACE_H
#define GINN_NODE_INPLACE_H

#include <ginn/node/common.h>
#include <ginn/node/data.h>
#include <ginn/node/layernorm.h>
#include <ginn/node/layout.h>
#include <ginn/nonlin.h>

namespace ginn {

// x *= val in place; the gradient is scaled in place on the way back
// (ginn/node/inplace.h:104-123).  The scaling is done when the value is first
// read (a Softmax behind a mask step takes it over, node/nlnode.h), at the
// latest when the forward pass of the Graph / LevelExecutor ends.
template <typename Scalar>
class InPlaceProdScalarNode : public BaseDataNode<Scalar>, public PendingInPlace {
  NodePtr<Scalar> in_;
  float val_;
  mutable bool pending_ = false;  // forward() has run, the scaling has not (PendingInPlace)
  bool skip_backward_ = false;

  void scale(Tensor<Scalar>& t) const {
    if (t.dev()->kind() == CPU)
      return host::scale_shift<Scalar>(static_cast<size_t>(t.size()), val_, 0.f, t.data(), t.data(), false);
    internal::require_gpu(t.dev(), "InPlaceProdScalar");
    GINN_HIP_CALL(ginn_hip_scale_shift(internal::ctx_of(t), dtype_of<Scalar>(), static_cast<size_t>(t.size()), val_,
                                       0.f, t.data(), t.data(), 0));
  }
  void forward_() override {
    pending_ = true;
    skip_backward_ = false;
  }
  void backward_() override {
    if (skip_backward_) {
      skip_backward_ = false;
      return;
    }
    if (in_->has_grad()) scale(in_->grad());
  }

 public:
  const Tensor<Scalar>& value() const override {
    if (pending_) {
      pending_ = false;
      scale(in_->value());
    }
    return std::as_const(*in_).value();
  }
  const Tensor<Scalar>& grad() const override { return std::as_const(*in_).grad(); }
  using Node<Scalar>::value;
  using Node<Scalar>::grad;
  Shape shape() const override { return in_->shape(); }
  DevPtr dev() const override { return in_->dev(); }
  bool has_grad() const override { return in_->has_grad(); }
  Step pending_step() const override { return Step::Scale; }
  bool pending() const override { return pending_; }
  void take_pending() override { pending_ = false; }
  float pending_value() const override { return val_; }
  BaseNode* pending_input() const override { return in_.get(); }
  void skip_next_backward() override { skip_backward_ = true; }
  void settle() override { (void)std::as_const(*this).value(); }
  // A skip that the pass it was meant for did not consume (a backward pass cut short, nodes run by
  // hand) must not reach the next one; the executors therefore call reset_grad() here in every pass.
  void reset_grad() override { skip_backward_ = false; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override { return false; }
  GINN_GRAD_IS_ALIAS_OF_BUT_FOR_RESET(in_)
  template <typename Val>
  InPlaceProdScalarNode(const NodePtr<Scalar>& in, Val val)
      : BaseDataNode<Scalar>({in}), in_(in), val_(static_cast<float>(val)) {}
  std::string name() const override { return "InPlaceProdScalar"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceProdScalar);

// Entries of x whose mask entry is 0 become mask_val; the mask is broadcast
// over the trailing dimensions in which it has extent 1.  Backward zeroes the
// gradient at the masked entries (ginn/node/inplace.h:152-212).
template <typename Scalar>
class InPlaceMaskNode : public BaseDataNode<Scalar>, public PendingInPlace {
  NodePtr<Scalar> in_, mask_;
  float mask_val_;
  mutable bool pending_ = false;  // forward() has run, the masking has not (PendingInPlace)
  bool skip_backward_ = false;

  void fill(Tensor<Scalar>& t, float v) const {
    const Size ms = mask_->value().size();
    if (t.dev()->kind() == CPU)
      return host::mask_fill<Scalar>(static_cast<size_t>(ms), static_cast<size_t>(t.size() / ms), mask_->value().data(),
                                     v, t.data());
    internal::require_gpu(t.dev(), "InPlaceMask");
    GINN_HIP_CALL(ginn_hip_mask_fill(internal::ctx_of(t), dtype_of<Scalar>(), static_cast<size_t>(ms),
                                     static_cast<size_t>(t.size() / ms), mask_->value().data(), v, t.data()));
  }
  void forward_() override {
    const Shape ms = mask_->value().shape(), is = in_->shape();  // shape(), not value(): a pending step below stays so
    GINN_ASSERT(ms.size() == is.size(), "InPlaceMask: mask and input ranks differ");
    size_t i = 0;
    while (i < is.size() && ms[i] == is[i]) ++i;
    for (; i < is.size(); ++i) GINN_ASSERT(ms[i] == 1, "Unexpected mask shape!");
    GINN_ASSERT(mask_->value().size() > 0);
    pending_ = true;
    skip_backward_ = false;
  }
  void backward_() override {
    if (skip_backward_) {
      skip_backward_ = false;
      return;
    }
    if (in_->has_grad()) fill(in_->grad(), 0.f);
  }

 public:
  const Tensor<Scalar>& value() const override {
    if (pending_) {
      pending_ = false;
      fill(in_->value(), mask_val_);  // in_->value() first runs a step pending below
    }
    return std::as_const(*in_).value();
  }
  const Tensor<Scalar>& grad() const override { return std::as_const(*in_).grad(); }
  using Node<Scalar>::value;
  using Node<Scalar>::grad;
  Shape shape() const override { return in_->shape(); }
  DevPtr dev() const override { return in_->dev(); }
  bool has_grad() const override { return in_->has_grad(); }
  Step pending_step() const override { return Step::Mask; }
  bool pending() const override { return pending_; }
  void take_pending() override { pending_ = false; }
  float pending_value() const override { return mask_val_; }
  BaseNode* pending_mask() const override { return mask_.get(); }
  BaseNode* pending_input() const override { return in_.get(); }
  void skip_next_backward() override { skip_backward_ = true; }
  void settle() override { (void)std::as_const(*this).value(); }
  // A skip that the pass it was meant for did not consume (a backward pass cut short, nodes run by
  // hand) must not reach the next one; the executors therefore call reset_grad() here in every pass.
  void reset_grad() override { skip_backward_ = false; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override { return false; }
  GINN_GRAD_IS_ALIAS_OF_BUT_FOR_RESET(in_)
  template <typename Val>
  InPlaceMaskNode(const NodePtr<Scalar>& in, const NodePtr<Scalar>& mask, Val mask_val)
      : BaseDataNode<Scalar>({in, mask}), in_(in), mask_(mask), mask_val_(static_cast<float>(mask_val)) {}
  std::string name() const override { return "InPlaceMask"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceMask);

// Aliasing boilerplate shared by the nodes below: value / gradient / has_grad
// are those of the node IN, and nothing is handed to the level executor.
#define GINN_INPLACE_ALIASES(IN)                                                               \
  const Tensor<Scalar>& value() const override { return std::as_const(*IN).value(); }          \
  const Tensor<Scalar>& grad() const override { return std::as_const(*IN).grad(); }            \
  using Node<Scalar>::value;                                                                   \
  using Node<Scalar>::grad;                                                                    \
  bool has_grad() const override { return IN->has_grad(); }                                    \
  GINN_GRAD_IS_ALIAS_OF(IN)                                                                    \
  bool describe_forward(std::vector<LaunchDesc>&) override { return false; }                   \
  bool describe_backward(std::vector<LaunchDesc>&) override { return false; }

// in_0 += in_1 + ...; the gradient of in_0 is this node's own, the others
// receive it (ginn/node/inplace.h:34-58).
template <typename Scalar>
class InPlaceAddNode : public AddNode<Scalar> {
 protected:
  using AddNode<Scalar>::ins_;
  void forward_() override {
    std::vector<const Tensor<Scalar>*> srcs;
    for (size_t i = 1; i < ins_.size(); ++i) srcs.push_back(&ins_[i]->value());
    if (!srcs.empty()) internal::add_tensors(ins_[0]->value(), srcs, true);
  }
  void backward_() override {
    for (size_t i = 1; i < ins_.size(); ++i)
      if (ins_[i]->has_grad()) internal::add_tensors(ins_[i]->grad(), {&grad()}, true);
  }

 public:
  using AddNode<Scalar>::AddNode;
  GINN_INPLACE_ALIASES(ins_[0])
  std::string name() const override { return "InPlaceAdd"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceAdd);

// x += val in place; the gradient passes through untouched (ginn/node/inplace.h:60-78).
template <typename Scalar>
class InPlaceAddScalarNode : public ScaleShiftNode<Scalar> {
 protected:
  using ScaleShiftNode<Scalar>::in_;
  void forward_() override {
    auto& x = in_->value();
    internal::require_gpu(x.dev(), "InPlaceAddScalar");
    GINN_HIP_CALL(ginn_hip_scale_shift(internal::ctx_of(x), dtype_of<Scalar>(), static_cast<size_t>(x.size()), 1.f,
                                       this->shift_, x.data(), x.data(), 0));
  }
  void backward_() override {}

 public:
  template <typename Val>
  InPlaceAddScalarNode(const NodePtr<Scalar>& in, Val val)
      : ScaleShiftNode<Scalar>(in, 1.f, static_cast<float>(Scalar(static_cast<float>(val))), "InPlaceAddScalar") {}
  GINN_INPLACE_ALIASES(in_)
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceAddScalar);

// a *= b in place.  a's old value is gone by the time of the backward pass, so
// db is formed from the product: db += dy * (value / b); da = dy * b
// (ginn/node/inplace.h:80-102).
template <typename Scalar>
class InPlaceCwiseProdNode : public CwiseProdNode<Scalar> {
 protected:
  using CwiseProdNode<Scalar>::a_;
  using CwiseProdNode<Scalar>::b_;
  void forward_() override {
    auto& a = a_->value();
    internal::require_gpu(a.dev(), "InPlaceCwiseProd");
    GINN_ASSERT(a.size() == b_->value().size(), "CwiseProd: operand sizes differ");
    GINN_HIP_CALL(ginn_hip_cwise_prod(internal::ctx_of(a), dtype_of<Scalar>(), static_cast<size_t>(a.size()), a.data(),
                                      b_->value().data(), a.data(), 0));
  }
  void backward_() override {
    const size_t n = static_cast<size_t>(grad().size());
    if (b_->has_grad())
      GINN_HIP_CALL(ginn_hip_elementwise(internal::ctx_of(grad()), dtype_of<Scalar>(), GINN_HIP_EW_DIV_MUL, n,
                                         grad().data(), a_->value().data(), b_->value().data(), b_->grad().data(), 1));
    if (a_->has_grad())
      GINN_HIP_CALL(ginn_hip_cwise_prod(internal::ctx_of(grad()), dtype_of<Scalar>(), n, grad().data(),
                                        b_->value().data(), a_->grad().data(), 0));
  }

 public:
  using CwiseProdNode<Scalar>::CwiseProdNode;
  GINN_INPLACE_ALIASES(a_)
  std::string name() const override { return "InPlaceCwiseProd"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceCwiseProd);

// Dropout over the input's own storage; the gradient is masked and scaled
// where it is (ginn/node/inplace.h:126-150).
template <typename Scalar>
class InPlaceDropoutNode : public DropoutNode<Scalar> {
 protected:
  using DropoutNode<Scalar>::in_;
  using DropoutNode<Scalar>::p_;
  using DropoutNode<Scalar>::mask_;
  void backward_() override {
    if (in_->has_grad() && p_ < 1.)
      GINN_HIP_CALL(ginn_hip_mask_scale(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                        static_cast<size_t>(grad().size()), this->scale(), grad().data(),
                                        reinterpret_cast<const unsigned char*>(mask_.data()), grad().data(), 0));
  }

 public:
  using DropoutNode<Scalar>::DropoutNode;
  GINN_INPLACE_ALIASES(in_)
  std::string name() const override { return "InPlaceDropout"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceDropout);

// LayerNorm over the input's own storage; the backward pass replaces the
// gradient (ginn/node/inplace.h:214-246).
template <typename Scalar>
class InPlaceLayerNormNode : public LayerNormNode<Scalar> {
 protected:
  using LayerNormNode<Scalar>::in_;
  using LayerNormNode<Scalar>::std_;
  void backward_() override {
    if (!in_->has_grad()) return;
    auto& y = value();
    GINN_HIP_CALL(ginn_hip_layernorm_bwd_assign(internal::ctx_of(y), dtype_of<Scalar>(), static_cast<int>(y.rows()),
                                                static_cast<int>(y.cols()), grad().data(), y.data(), std_.data(),
                                                grad().data()));
  }

 public:
  using LayerNormNode<Scalar>::LayerNormNode;
  GINN_INPLACE_ALIASES(in_)
  bool may_postpone() const override { return false; }
  std::string name() const override { return "InPlaceLayerNorm"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlaceLayerNorm);

// Permutes the axes of the input inside the input's storage: value() and
// grad() are views of it under the permuted shape (ginn/node/inplace.h:248-309).
template <typename Scalar>
class InPlacePermuteNode : public PermuteNode<Scalar> {
 protected:
  using PermuteNode<Scalar>::in_;
  using PermuteNode<Scalar>::indices_;
  void forward_() override {
    const Shape s = in_->shape();
    this->check_permutation(s);
    Tensor<Scalar> tmp(in_->value().dev(), PermuteNode<Scalar>::permute(s, indices_));
    PermuteNode<Scalar>::run(in_->value(), s, indices_, tmp, false);
    this->value().map(in_->value(), tmp.shape());
    this->value() = tmp;  // same size: copies into the input's storage
  }

 public:
  InPlacePermuteNode(const NodePtr<Scalar>& in, Shape indices) : PermuteNode<Scalar>(in, std::move(indices)) {
    this->overwrite_ = true;
  }
  bool has_grad() const override { return in_->has_grad(); }
  bool owns_grad() const override { return false; }  // the input's gradient under the permuted shape
  void init_grad() override {
    if (this->has_grad()) this->grad().map(in_->grad(), PermuteNode<Scalar>::permute(in_->shape(), indices_));
  }
  void reset_grad() override { init_grad(); }
  bool describe_forward(std::vector<LaunchDesc>&) override { return false; }
  bool describe_backward(std::vector<LaunchDesc>&) override { return false; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    init_grad();
    return true;
  }
  std::string name() const override { return "InPlacePermute"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(InPlacePermute);
template <typename NodePtrType>
auto InPlacePermute(NodePtrType x, std::initializer_list<Size> indices) {
  return InPlacePermute(std::move(x), Shape(indices));
}

#undef GINN_INPLACE_ALIASES

}  // namespace ginn

#endif  // GINN_NODE_INPLACE_H
