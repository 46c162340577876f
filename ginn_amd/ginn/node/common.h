// Arithmetic nodes used around the product path (ginn/node/common.h): N-ary
// Add, Subtract, CwiseProd, CwiseProdAdd, CwiseMax, ProdScalar, AddScalar,
// SubtractScalar, Dropout and the operator sugar for them.
#ifndef GINN_NODE_COMMON_H
#define GINN_NODE_COMMON_H

#include <ginn/node/data.h>
#include <ginn/node/layernorm.h>
#include <ginn/nonlin.h>

namespace ginn {

namespace internal {

// dst (+)= sum of srcs, in groups of eight per launch.
template <typename Scalar>
void add_tensors(Tensor<Scalar>& dst, const std::vector<const Tensor<Scalar>*>& srcs, bool accumulate) {
  const size_t n = static_cast<size_t>(dst.size());
  if (dst.dev()->kind() == CPU) {
    std::vector<const Scalar*> p;
    for (auto* s : srcs) {
      GINN_ASSERT(s->size() == dst.size(), "Add: operand sizes differ");
      p.push_back(s->data());
    }
    if constexpr (is_floating_point_v<Scalar>) host::add_n<Scalar>(n, p, dst.data(), accumulate);
    else GINN_THROW("Add on cpu(): floating-point scalars only");
    return;
  }
  require_gpu(dst.dev(), "Add");
  for (size_t i = 0; i < srcs.size(); i += 8) {
    const int count = static_cast<int>(std::min<size_t>(8, srcs.size() - i));
    const void* p[8];
    for (int k = 0; k < count; ++k) {
      GINN_ASSERT(srcs[i + k]->size() == dst.size(), "Add: operand sizes differ");
      p[k] = srcs[i + k]->data();
    }
    GINN_HIP_CALL(ginn_hip_add_n(ctx_of(dst), arith_dtype_of<Scalar>(), n, count, p, dst.data(),
                                 (accumulate || i > 0) ? 1 : 0));
  }
}

}  // namespace internal

// value = in_0 + ... + in_{N-1}; backward adds the gradient to every input
// (ginn/node/common.h:97-157).
template <typename Scalar>
class AddNode : public BaseDataNode<Scalar> {
 protected:
  std::vector<NodePtr<Scalar>> ins_;

  void forward_() override {
    value().resize(ins_[0]->value().shape());
    std::vector<const Tensor<Scalar>*> srcs;
    for (auto& in : ins_) srcs.push_back(&in->value());
    internal::add_tensors(value(), srcs, false);
  }
  void backward_() override {
    for (auto& in : ins_) {
      if (!in->has_grad()) continue;
      const bool fresh = in->take_lazy_zero();
      internal::add_tensors(in->grad(), {&grad()}, !fresh);
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }

  bool describe_forward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    value().resize(ins_[0]->value().shape());
    for (size_t i = 0; i < ins_.size(); i += 3) {
      LaunchDesc d;
      d.dtype = arith_dtype_of<Scalar>();
      d.kind = GINN_HIP_MULTI_SUM;
      d.accumulate = i > 0;
      d.n = static_cast<size_t>(value().size());
      d.dst = value().data();
      for (size_t k = 0; k < 3 && i + k < ins_.size(); ++k) {
        GINN_ASSERT(ins_[i + k]->value().size() == value().size(), "Add: operand sizes differ");
        d.src[k] = ins_[i + k]->value().data();
      }
      out.push_back(d);
    }
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    for (auto& in : ins_) {
      if (!in->has_grad()) continue;
      LaunchDesc d;
      d.dtype = arith_dtype_of<Scalar>();
      d.kind = GINN_HIP_MULTI_SUM;
      d.accumulate = !in->take_lazy_zero();
      d.n = static_cast<size_t>(grad().size());
      d.dst = in->grad().data();
      d.src[0] = grad().data();
      out.push_back(d);
    }
    return true;
  }
  AddNode(const std::vector<NodePtr<Scalar>>& ins) : BaseDataNode<Scalar>(ins), ins_(ins) {}
  template <typename... Args>
  AddNode(const NodePtr<Scalar>& in, const Args&... args) : AddNode(std::vector<NodePtr<Scalar>>{in, args...}) {}

  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    BaseNode::ins_ = ins;
    ins_ = derived_cast<Node<Scalar>>(ins);
  }
  std::string name() const override { return "Add"; }
};

GINN_MAKE_SCALAR_FORWARDING_FACTORY(Add);

// value = a (*) b; backward da += dy (*) b, db += dy (*) a (ginn/node/common.h:233-262).
template <typename Scalar>
class CwiseProdNode : public BaseDataNode<Scalar> {
 protected:
  NodePtr<Scalar> a_, b_;

  void run(Tensor<Scalar>& dst, const Tensor<Scalar>& x, const Tensor<Scalar>& y, bool acc) {
    if (dst.dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>)
        return host::cwise_prod<Scalar>(static_cast<size_t>(dst.size()), x.data(), y.data(), dst.data(), acc);
    }
    internal::require_gpu(dst.dev(), "CwiseProd");
    GINN_HIP_CALL(ginn_hip_cwise_prod(internal::ctx_of(dst), arith_dtype_of<Scalar>(), static_cast<size_t>(dst.size()),
                                      x.data(), y.data(), dst.data(), acc ? 1 : 0));
  }
  void forward_() override {
    GINN_ASSERT(a_->value().size() == b_->value().size(), "CwiseProd: operand sizes differ");
    value().resize(a_->value().shape());
    run(value(), a_->value(), b_->value(), false);
  }
  void backward_() override {
    if (a_->has_grad()) {
      const bool fresh = a_->take_lazy_zero();
      run(a_->grad(), grad(), b_->value(), !fresh);
    }
    if (b_->has_grad()) {
      const bool fresh = b_->take_lazy_zero();
      run(b_->grad(), grad(), a_->value(), !fresh);
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }
  LaunchDesc prod_desc(Scalar* dst, const Scalar* x, const Scalar* y, bool accumulate) const {
    LaunchDesc d;
    d.dtype = arith_dtype_of<Scalar>();
    d.kind = GINN_HIP_MULTI_PROD;
    d.accumulate = accumulate;
    d.n = static_cast<size_t>(value().size());
    d.dst = dst;
    d.src[0] = x;
    d.src[1] = y;
    return d;
  }
  bool describe_forward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    GINN_ASSERT(a_->value().size() == b_->value().size(), "CwiseProd: operand sizes differ");
    value().resize(a_->value().shape());
    out.push_back(prod_desc(value().data(), a_->value().data(), b_->value().data(), false));
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    if (a_->has_grad()) {
      const bool fresh = a_->take_lazy_zero();
      out.push_back(prod_desc(a_->grad().data(), grad().data(), b_->value().data(), !fresh));
    }
    if (b_->has_grad()) {
      const bool fresh = b_->take_lazy_zero();
      out.push_back(prod_desc(b_->grad().data(), grad().data(), a_->value().data(), !fresh));
    }
    return true;
  }
  CwiseProdNode(const NodePtr<Scalar>& a, const NodePtr<Scalar>& b) : BaseDataNode<Scalar>({a, b}), a_(a), b_(b) {}
  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() == 2);
    BaseNode::ins_ = ins;
    a_ = dynamic_ptr_cast<Node<Scalar>>(ins[0]);
    b_ = dynamic_ptr_cast<Node<Scalar>>(ins[1]);
  }
  std::string name() const override { return "CwiseProd"; }
};

GINN_MAKE_SCALAR_FORWARDING_FACTORY(CwiseProd);

// value = alpha * x + shift: ProdScalar (shift = 0) and AddScalar (alpha = 1).
template <typename Scalar>
class ScaleShiftNode : public BaseDataNode<Scalar> {
 protected:
  NodePtr<Scalar> in_;
  float alpha_, shift_;
  const char* name_;

  void forward_() override {
    value().resize(in_->value().shape());
    if (this->dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>)
        return host::scale_shift<Scalar>(static_cast<size_t>(value().size()), alpha_, shift_, in_->value().data(),
                                        value().data(), false);
    }
    internal::require_gpu(this->dev(), name_);
    GINN_HIP_CALL(ginn_hip_scale_shift(internal::ctx_of(value()), arith_dtype_of<Scalar>(),
                                       static_cast<size_t>(value().size()), alpha_, shift_, in_->value().data(),
                                       value().data(), 0));
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    const bool fresh = in_->take_lazy_zero();
    if (this->dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>)
        return host::scale_shift<Scalar>(static_cast<size_t>(grad().size()), alpha_, 0.f, grad().data(),
                                        in_->grad().data(), !fresh);
    }
    GINN_HIP_CALL(ginn_hip_scale_shift(internal::ctx_of(grad()), arith_dtype_of<Scalar>(),
                                       static_cast<size_t>(grad().size()), alpha_, 0.f, grad().data(),
                                       in_->grad().data(), fresh ? 0 : 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }
  ScaleShiftNode(const NodePtr<Scalar>& in, float alpha, float shift, const char* name)
      : BaseDataNode<Scalar>({in}), in_(in), alpha_(alpha), shift_(shift), name_(name) {}
  std::string name() const override { return name_; }
};

// value = a (*) (b + multiplier_bias) + c.  b and c either have a's shape or
// are rank-1 vectors of a's row count, applied to every column -- the gamma /
// beta step after LayerNorm (ginn/node/common.h:245-316).
template <typename Scalar>
class CwiseProdAddNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> a_, b_, c_;
  bool broadcast_ = false;
  float multiplier_bias_;

  void forward_() override {
    // shape(), not value(): a LayerNorm in front that has not run yet stays so
    const Shape s0 = a_->shape(), s1 = b_->value().shape(), s2 = c_->value().shape();
    if (s0 == s1 && s1 == s2) {
      broadcast_ = false;
    } else if (s1.size() == 1 && s2.size() == 1) {
      broadcast_ = true;
      GINN_ASSERT(s0[0] == s1[0] && s1[0] == s2[0], "Unexpected shapes for CwiseProdAdd!");
    } else {
      GINN_THROW("Unexpected shapes for CwiseProdAdd!");
    }
    value().resize(s0);
    if (this->dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>) {
        auto& a = a_->value();
        return host::cwise_prod_add_forward<Scalar>(static_cast<int>(a.rows()), static_cast<int>(a.cols()), a.data(),
                                                    b_->value().data(), c_->value().data(), multiplier_bias_,
                                                    broadcast_, value().data());
      }
    }
    internal::require_gpu(this->dev(), "CwiseProdAdd");
    // Right behind a LayerNorm whose kernel has not run yet: normalisation and
    // the gamma / beta step as one pass (same values).
    if (LayerNormNode<Scalar>* ln = broadcast_ ? layer_norm() : nullptr; ln && ln->pending_) {
      ln->pending_ = false;
      auto& x = ln->in_->value();
      GINN_HIP_CALL(ginn_hip_layernorm_affine_fwd(
          internal::ctx_of(x), arith_dtype_of<Scalar>(), static_cast<int>(x.rows()), static_cast<int>(x.cols()), x.data(),
          ln->eps_, b_->value().data(), c_->value().data(), multiplier_bias_, ln->raw_value().data(), ln->std_.data(),
          value().data()));
      return;
    }
    auto& a = a_->value();
    GINN_HIP_CALL(ginn_hip_cwise_prod_add_fwd(internal::ctx_of(a), arith_dtype_of<Scalar>(), static_cast<int>(a.rows()),
                                              static_cast<int>(a.cols()), a.data(), b_->value().data(),
                                              c_->value().data(), multiplier_bias_, broadcast_ ? 1 : 0,
                                              value().data()));
  }
  void backward_() override {
    auto& a = a_->value();
    if (this->dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>) {
        const bool fresh = a_->has_grad() && a_->take_lazy_zero();
        return host::cwise_prod_add_backward<Scalar>(
            static_cast<int>(a.rows()), static_cast<int>(a.cols()), grad().data(), a.data(), b_->value().data(),
            multiplier_bias_, broadcast_, a_->has_grad() ? a_->grad().data() : nullptr, !fresh,
            b_->has_grad() ? b_->grad().data() : nullptr, c_->has_grad() ? c_->grad().data() : nullptr);
      }
    }
    internal::PostponeFolds later(internal::ctx_of(a), *b_, *c_);  // scale / shift gradients: complete at the pass's end
    // A flagged gradient of a means: this node is its only user and overwrites.
    const bool fresh = a_->has_grad() && a_->take_lazy_zero();
    LayerNormNode<Scalar>* ln = fresh && broadcast_ && b_->has_grad() == c_->has_grad() ? layer_norm() : nullptr;
    if (ln) {
      // ... and behind a LayerNorm nobody else will read that gradient either: both
      // backward steps as one pass, the LayerNorm node skips its own.
      auto& x = ln->in_;
      const bool x_fresh = x->has_grad() && x->take_lazy_zero();
      GINN_HIP_CALL(ginn_hip_layernorm_affine_bwd(
          internal::ctx_of(a), arith_dtype_of<Scalar>(), static_cast<int>(a.rows()), static_cast<int>(a.cols()),
          grad().data(), a.data(), ln->std_.data(), b_->value().data(), multiplier_bias_,
          x->has_grad() ? x->grad().data() : nullptr, x_fresh ? 0 : 1, b_->has_grad() ? b_->grad().data() : nullptr,
          c_->has_grad() ? c_->grad().data() : nullptr));
      ln->skip_backward_ = true;
      return;
    }
    GINN_HIP_CALL((fresh ? ginn_hip_cwise_prod_add_bwd_assign : ginn_hip_cwise_prod_add_bwd)(
        internal::ctx_of(a), arith_dtype_of<Scalar>(), static_cast<int>(a.rows()), static_cast<int>(a.cols()),
        grad().data(), a.data(), b_->value().data(), multiplier_bias_, broadcast_ ? 1 : 0,
        a_->has_grad() ? a_->grad().data() : nullptr, b_->has_grad() ? b_->grad().data() : nullptr,
        c_->has_grad() ? c_->grad().data() : nullptr));
  }
  // The LayerNorm this node follows directly, if any (not one that normalises in place).
  LayerNormNode<Scalar>* layer_norm() const {
    if constexpr (is_floating_point_v<Scalar>) {
      auto* ln = dynamic_cast<LayerNormNode<Scalar>*>(a_.get());
      return ln && ln->may_postpone() ? ln : nullptr;
    } else {
      return nullptr;
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  template <typename Bias = Scalar>
  CwiseProdAddNode(const NodePtr<Scalar>& a, const NodePtr<Scalar>& b, const NodePtr<Scalar>& c,
                   Bias multiplier_bias = Bias(0))
      : BaseDataNode<Scalar>({a, b, c}), a_(a), b_(b), c_(c),
        multiplier_bias_(static_cast<float>(multiplier_bias)) {}
  // The gradient of a is overwritten when it holds no value yet; b and c are added to.
  BaseNode::GradUse grad_use(size_t index) const override {
    return index == 0 ? BaseNode::GradUse::Overwrites : BaseNode::GradUse::Accumulates;
  }
  std::string name() const override { return "CwiseProdAdd"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(CwiseProdAdd);

// The scalar operand is held in the node's scalar type, as in the reference
// (`val_(Scalar(b))`, ginn/node/common.h:45-46,218-219): for Half, x * 3.14
// multiplies by the nearest Half.
template <typename NodeT>
auto ProdScalar(const Ptr<NodeT>& x, double a) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<ScaleShiftNode<Scalar>>(NodePtr<Scalar>(x), static_cast<float>(Scalar(static_cast<float>(a))), 0.f,
                                          "ProdScalar");
}
template <typename NodeT>
auto AddScalar(const Ptr<NodeT>& x, double s) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<ScaleShiftNode<Scalar>>(NodePtr<Scalar>(x), 1.f, static_cast<float>(Scalar(static_cast<float>(s))),
                                          "AddScalar");
}
// a - x for a scalar on the left (ginn/node/common.h:55-95).
template <typename NodeT>
auto SubtractScalar(double a, const Ptr<NodeT>& x) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<ScaleShiftNode<Scalar>>(NodePtr<Scalar>(x), -1.f, static_cast<float>(Scalar(static_cast<float>(a))),
                                          "SubtractScalar");
}

// value = left - right; backward left += dy, right -= dy (ginn/node/common.h:162-187).
template <typename Scalar>
class SubtractNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> left_, right_;

  void forward_() override {
    internal::require_gpu(this->dev(), "Subtract");
    GINN_ASSERT(left_->value().size() == right_->value().size(), "Subtract: operand sizes differ");
    value().resize(left_->value().shape());
    GINN_HIP_CALL(ginn_hip_elementwise(internal::ctx_of(value()), arith_dtype_of<Scalar>(), GINN_HIP_EW_SUB,
                                       static_cast<size_t>(value().size()), left_->value().data(),
                                       right_->value().data(), nullptr, value().data(), 0));
  }
  void backward_() override {
    if (left_->has_grad()) internal::add_tensors(left_->grad(), {&grad()}, true);
    if (right_->has_grad())
      GINN_HIP_CALL(ginn_hip_scale_shift(internal::ctx_of(grad()), arith_dtype_of<Scalar>(),
                                         static_cast<size_t>(grad().size()), -1.f, 0.f, grad().data(),
                                         right_->grad().data(), 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  SubtractNode(const NodePtr<Scalar>& a, const NodePtr<Scalar>& b) : BaseDataNode<Scalar>({a, b}), left_(a), right_(b) {}
  std::string name() const override { return "Subtract"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Subtract);

// value = elementwise maximum of the inputs; the gradient goes to every input
// that equals the maximum (ginn/node/common.h:319-357).
template <typename Scalar>
class CwiseMaxNode : public BaseDataNode<Scalar> {
  std::vector<NodePtr<Scalar>> ins_;

  void forward_() override {
    internal::require_gpu(this->dev(), "CwiseMax");
    value().resize(ins_[0]->value().shape());
    value() = ins_[0]->value();
    for (size_t i = 1; i < ins_.size(); ++i) {
      GINN_ASSERT(ins_[i]->value().size() == value().size(), "CwiseMax: operand sizes differ");
      GINN_HIP_CALL(ginn_hip_elementwise(internal::ctx_of(value()), arith_dtype_of<Scalar>(), GINN_HIP_EW_MAX,
                                         static_cast<size_t>(value().size()), value().data(),
                                         ins_[i]->value().data(), nullptr, value().data(), 0));
    }
  }
  void backward_() override {
    for (auto& in : ins_)
      if (in->has_grad())
        GINN_HIP_CALL(ginn_hip_elementwise(internal::ctx_of(grad()), arith_dtype_of<Scalar>(), GINN_HIP_EW_EQ_MUL,
                                           static_cast<size_t>(grad().size()), grad().data(), in->value().data(),
                                           value().data(), in->grad().data(), 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  CwiseMaxNode(const std::vector<NodePtr<Scalar>>& ins) : BaseDataNode<Scalar>(ins), ins_(ins) {}
  template <typename... Args>
  CwiseMaxNode(const NodePtr<Scalar>& in, const Args&... args)
      : CwiseMaxNode(std::vector<NodePtr<Scalar>>{in, args...}) {}
  std::string name() const override { return "CwiseMax"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(CwiseMax);

// value = x * mask / (1 - p) with mask ~ Bernoulli(1 - p), drawn anew at every
// forward pass (ginn/node/common.h:359-402).  The mask comes from a
// counter-based generator on the device; seeds advance process-wide.
template <typename Scalar>
class DropoutNode : public BaseDataNode<Scalar> {
  static_assert(is_floating_point_v<Scalar>, "Dropout scalar needs to be floating point because of scaling!");

 protected:
  NodePtr<Scalar> in_;
  Real p_;
  Tensor<bool> mask_;

  static unsigned long long next_seed() {
    static std::atomic<unsigned long long> s{0x2545f4914f6cdd1dull};
    return s += 0x9e3779b97f4a7c15ull;
  }
  float scale() const { return static_cast<float>(Scalar(static_cast<float>(1. / (1. - p_)))); }

  void forward_() override {
    internal::require_gpu(this->dev(), "Dropout");
    auto& x = in_->value();
    value().resize(x.shape());
    if (p_ == 1.) {
      value().set_zero();
      return;
    }
    mask_.resize(x.shape());
    const size_t n = static_cast<size_t>(x.size());
    GINN_HIP_CALL(ginn_hip_dropout_mask(internal::ctx_of(x), n, static_cast<float>(p_), next_seed(),
                                        reinterpret_cast<unsigned char*>(mask_.data())));
    GINN_HIP_CALL(ginn_hip_mask_scale(internal::ctx_of(x), dtype_of<Scalar>(), n, scale(), x.data(),
                                      reinterpret_cast<const unsigned char*>(mask_.data()), value().data(), 0));
  }
  void backward_() override {
    if (in_->has_grad() && p_ < 1.)
      GINN_HIP_CALL(ginn_hip_mask_scale(internal::ctx_of(grad()), dtype_of<Scalar>(),
                                        static_cast<size_t>(grad().size()), scale(), grad().data(),
                                        reinterpret_cast<const unsigned char*>(mask_.data()), in_->grad().data(), 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  DropoutNode(const NodePtr<Scalar>& in, Real p)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{in}), in_(in), p_(p), mask_(in->dev()) {
    GINN_ASSERT(p_ >= 0 && p_ <= 1, "Dropout probability is not in [0, 1]!");
  }
  const Tensor<bool>& mask() const { return mask_; }
  std::string name() const override { return "Dropout"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Dropout);

// Operator sugar (ginn/node/common.h:404-479): node (+|-) node, node (+|-|*) scalar,
// scalar (+|-|*) node, -node.
template <typename Left, typename Right,
          typename = std::enable_if_t<is_node_ptr_v<Left> || is_node_ptr_v<Right>>>
auto operator+(const Left& a, const Right& b) {
  if constexpr (is_node_ptr_v<Left> && is_node_ptr_v<Right>) {
    using Scalar = typename Left::element_type::Scalar;
    return Add(NodePtr<Scalar>(a), NodePtr<Scalar>(b));
  } else if constexpr (is_node_ptr_v<Left>) {
    return AddScalar(a, static_cast<double>(b));
  } else {
    return AddScalar(b, static_cast<double>(a));
  }
}
template <typename Left, typename Right,
          typename = std::enable_if_t<is_node_ptr_v<Left> || is_node_ptr_v<Right>>>
auto operator-(const Left& a, const Right& b) {
  if constexpr (is_node_ptr_v<Left> && is_node_ptr_v<Right>) {
    using Scalar = typename Left::element_type::Scalar;
    return Subtract(NodePtr<Scalar>(a), NodePtr<Scalar>(b));
  } else if constexpr (is_node_ptr_v<Left>) {
    return AddScalar(a, -static_cast<double>(b));
  } else {
    return SubtractScalar(static_cast<double>(a), b);
  }
}
template <typename NodeT>
auto operator-(const Ptr<NodeT>& in) {
  return ProdScalar(in, -1.);
}
template <typename Left, typename Right,
          typename = std::enable_if_t<is_node_ptr_v<Left> != is_node_ptr_v<Right>>>
auto operator*(const Left& a, const Right& b) {
  if constexpr (is_node_ptr_v<Left>) return ProdScalar(a, static_cast<double>(b));
  else return ProdScalar(b, static_cast<double>(a));
}

}  // namespace ginn

#endif  // GINN_NODE_COMMON_H
