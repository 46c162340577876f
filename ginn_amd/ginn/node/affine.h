// AffineNode: Y = f(sum_i A_i * B_i + bias)  (ginn/node/affine.h:28-233).
//
// Forward is one call: the bias broadcast, the accumulating products and the
// nonlinearity of the reference become the epilogue of the last product
// kernel.  The pre-activation is kept only when the nonlinearity's backward
// needs its input.  Backward: dpre = f'(.) * dY and dbias += rowsum(dpre) in
// one pass, then per pair dB += A^T dpre and dA += dpre B^T.
#ifndef GINN_NODE_AFFINE_H
#define GINN_NODE_AFFINE_H

#include <optional>

#include <ginn/node/data.h>
#include <ginn/nonlin.h>
#include <ginn/prod.h>

namespace ginn {

template <typename Scalar>
class AffineNode : public BaseDataNode<Scalar> {
  std::vector<NodePtr<Scalar>> ins_;  // [A0, B0, A1, B1, ..., bias]
  Tensor<Scalar> preactiv_, dpreactiv_;
  std::unique_ptr<NonlinOp<Scalar>> nonlin_;

  void check_arity() const {
    GINN_ASSERT(ins_.size() > 0);
    GINN_ASSERT(ins_.size() % 2);  // pairs plus the bias
  }

  // On cpu(): the reference's own sequence (ginn/node/affine.h:35-77) -- bias broadcast, one accumulating
  // product per pair, the nonlinearity -- in the host layer's loops.
  void forward_cpu() {
    auto& bias = ins_.back()->value();
    Shape out = ins_[1]->value().shape();
    out[0] = ins_[0]->value().rows();
    const Size m = out[0];
    GINN_ASSERT(bias.size() == m, "Affine bias must have one entry per output row!");
    const bool keep_pre = nonlin_->backward_requires_input();
    value().resize(out);
    Tensor<Scalar>& pre = keep_pre ? preactiv_ : value();
    if (keep_pre) preactiv_.resize(out);
    const Size n = pre.cols();
    for (Size c = 0; c < n; ++c)
      for (Size r = 0; r < m; ++r) pre.data()[c * m + r] = bias.data()[r];
    for (size_t i = 0; i + 1 < ins_.size(); i += 2) {
      GINN_ASSERT(ins_[i]->value().shape().size() == 2);
      internal::cpu_prod(pre, ins_[i]->value(), ins_[i + 1]->value(), internal::ProdResult::Add);
    }
    if (!nonlin_->is_identity()) nonlin_->forward(value(), pre);
  }
  void backward_cpu() {
    using namespace internal;
    const bool identity = nonlin_->is_identity();
    Tensor<Scalar>& daffine = identity ? grad() : dpreactiv_;
    if (!identity) {
      dpreactiv_.resize(grad().shape());
      nonlin_->backward(dpreactiv_, grad(), preactiv_, value(), false);
    }
    auto& bias = ins_.back();
    const Size m = grad().rows(), n = grad().cols();
    if (bias->has_grad()) {
      const bool fresh = bias->take_lazy_zero();
      Scalar* db = bias->grad().data();
      for (Size r = 0; r < m; ++r) {
        float s = fresh ? 0.f : static_cast<float>(db[r]);
        for (Size c = 0; c < n; ++c) s += static_cast<float>(daffine.data()[c * m + r]);
        db[r] = Scalar(s);
      }
    }
    for (size_t i = 0; i + 1 < ins_.size(); i += 2) {
      auto &a = ins_[i], &b = ins_[i + 1];
      if (b->has_grad())
        cpu_prod(b->grad(), a->value(), daffine, b->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::First);
      if (a->has_grad())
        cpu_prod(a->grad(), daffine, b->value(), a->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::Second);
    }
  }

  void forward_() override {
    if (dev()->kind() == CPU) return forward_cpu();
    internal::require_gpu(dev(), "Affine");
    auto& a0 = ins_[0]->value();
    auto& b0 = ins_[1]->value();
    auto& bias = ins_.back()->value();
    GINN_ASSERT(a0.shape().size() == 2);
    Shape out = b0.shape();
    out[0] = a0.rows();
    const bool keep_pre = nonlin_->backward_requires_input();
    if (keep_pre) preactiv_.resize(out);
    value().resize(out);

    const int pairs = static_cast<int>(ins_.size() / 2);
    const Size m = a0.rows(), n = b0.cols();
    std::vector<const void*> W(pairs), X(pairs);
    std::vector<int> K(pairs);
    for (int p = 0; p < pairs; ++p) {
      auto& a = ins_[2 * p]->value();
      auto& b = ins_[2 * p + 1]->value();
      GINN_ASSERT(a.shape().size() == 2);
      GINN_ASSERT(a.rows() == m);
      GINN_ASSERT(a.cols() == b.rows());
      GINN_ASSERT(b.cols() == n);
      W[p] = a.data();
      X[p] = b.data();
      K[p] = static_cast<int>(a.cols());
    }
    GINN_ASSERT(bias.size() == m, "Affine bias must have one entry per output row!");
    GINN_HIP_CALL(ginn_hip_affine_fwd(internal::ctx_of(value()), dtype_of<Scalar>(), nonlin_->code(),
                                      static_cast<int>(m), static_cast<int>(n), pairs, W.data(), X.data(),
                                      K.data(), bias.data(), keep_pre ? preactiv_.data() : nullptr,
                                      value().data()));
  }

  static constexpr double kBesideRowSum = 1048576.;  // elements from which a row sum is worth a second stream

  void backward_() override {
    using namespace internal;
    if (dev()->kind() == CPU) return backward_cpu();
    const bool identity = nonlin_->is_identity();
    Tensor<Scalar>& daffine = identity ? grad() : dpreactiv_;
    if (!identity) dpreactiv_.resize(grad().shape());
    auto& bias = ins_.back();
    const Size m = grad().rows(), n = grad().cols();
    // Without an activation this call is the row sum for the bias gradient alone and nothing in the
    // pass waits for it: a large one runs beside the pass like the weight gradients below (and folds
    // at once there: the folds that wait for the end of the pass are flushed on the pass's own stream).
    ginn_hip_ctx* pre_ctx = ctx_of(grad());
    if (identity && bias->has_grad() && static_cast<double>(m) * static_cast<double>(n) >= kBesideRowSum)
      pre_ctx = BesidePass::ctx_for(*bias, dev(), BesidePass::kWorthIt);
    const bool beside = pre_ctx != ctx_of(grad());
    std::optional<PostponeFolds> later;  // the bias gradient is complete when the pass ends
    if (!beside) later.emplace(pre_ctx, *bias);
    GINN_HIP_CALL(ginn_hip_affine_bwd_pre(pre_ctx, dtype_of<Scalar>(), nonlin_->code(),
                                          static_cast<int>(m), static_cast<int>(n), grad().data(),
                                          value().data(), preactiv_.size() > 0 ? preactiv_.data() : nullptr,
                                          identity ? nullptr : dpreactiv_.data(),
                                          bias->has_grad() ? bias->grad().data() : nullptr));
    // The gradients the nodes below wait for first; those of leaves (weights) beside the pass:
    // daffine is this node's gradient or a buffer it keeps, unchanged until the next pass.
    for (const bool leaves : {false, true}) {
      for (size_t i = 0; i + 1 < ins_.size(); i += 2) {
        auto &a = ins_[i], &b = ins_[i + 1];
        const double flops = 2.0 * static_cast<double>(m) * static_cast<double>(n) * static_cast<double>(a->value().cols());
        if (b->has_grad() && b->inputs().empty() == leaves) {
          const bool fresh = b->take_lazy_zero();
          ginn_hip_ctx* where = BesidePass::ctx_for(*b, dev(), flops);
          gpu_prod(where, b->grad(), a->value(), daffine, fresh ? ProdResult::Assign : ProdResult::Add,
                   ProdTranspose::First);
        }
        if (a->has_grad() && a->inputs().empty() == leaves) {
          const bool fresh = a->take_lazy_zero();
          ginn_hip_ctx* where = BesidePass::ctx_for(*a, dev(), flops);
          gpu_prod(where, a->grad(), daffine, b->value(), fresh ? ProdResult::Assign : ProdResult::Add,
                   ProdTranspose::Second);
        }
      }
    }
  }

 public:
  using BaseDataNode<Scalar>::dev;
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;

  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    BaseNode::ins_ = ins;
    ins_ = derived_cast<Node<Scalar>>(ins);
  }

  template <typename NonlinType,
            typename = std::enable_if_t<std::is_base_of_v<NonlinOp<Scalar>, NonlinType>>>
  AffineNode(NonlinType nonlin, const std::vector<NodePtr<Scalar>>& ins)
      : BaseDataNode<Scalar>(ins),
        ins_(ins),
        preactiv_(dev()),
        dpreactiv_(dev()),
        nonlin_(std::make_unique<NonlinType>(nonlin)) {
    check_arity();
  }
  AffineNode(std::unique_ptr<NonlinOp<Scalar>> nonlin, const std::vector<NodePtr<Scalar>>& ins)
      : BaseDataNode<Scalar>(ins), ins_(ins), preactiv_(dev()), dpreactiv_(dev()), nonlin_(std::move(nonlin)) {
    check_arity();
  }
  AffineNode(const std::vector<NodePtr<Scalar>>& ins) : AffineNode(IdentityOp<Scalar>(), ins) {}

  template <typename... Args>
  AffineNode(const NodePtr<Scalar>& in, Args&&... args)
      : AffineNode(std::vector<NodePtr<Scalar>>({in, args...})) {}
  template <typename NonlinType, typename... Args,
            typename = std::enable_if_t<std::is_base_of_v<NonlinOp<Scalar>, NonlinType>>>
  AffineNode(NonlinType nonlin, const NodePtr<Scalar>& in, Args&&... args)
      : AffineNode(nonlin, std::vector<NodePtr<Scalar>>({in, args...})) {}

  const NonlinOp<Scalar>& nonlin() const { return *nonlin_; }
  // Products overwrite; the bias gradient is added to.
  BaseNode::GradUse grad_use(size_t index) const override {
    return index + 1 < ins_.size() ? BaseNode::GradUse::Overwrites : BaseNode::GradUse::Accumulates;
  }
  std::string name() const override { return "AffineNode"; }
};

// Factories (ginn/node/affine.h:184-233).
template <typename Scalar>
auto Affine(const std::vector<NodePtr<Scalar>>& ins) {
  return make_ptr<AffineNode<Scalar>>(ins);
}
template <typename NodeT, typename... Args, typename = std::enable_if_t<std::is_base_of_v<BaseNode, NodeT>>>
auto Affine(Ptr<NodeT> in, Args&&... args) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<AffineNode<Scalar>>(NodePtr<Scalar>(in), NodePtr<Scalar>(std::forward<Args>(args))...);
}
template <typename NodeT, typename NonlinType, typename... Args,
          typename = std::enable_if_t<std::is_base_of_v<NonlinOp<typename NodeT::Scalar>, NonlinType>>>
auto Affine(NonlinType nonlin, Ptr<NodeT> in, Args&&... args) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<AffineNode<Scalar>>(nonlin, NodePtr<Scalar>(in), NodePtr<Scalar>(std::forward<Args>(args))...);
}
template <template <typename> typename Nonlin, typename NodeT, typename... Args>
auto Affine(Ptr<NodeT> in, Args&&... args) {
  using Scalar = typename NodeT::Scalar;
  return make_ptr<AffineNode<Scalar>>(Nonlin<Scalar>(), NodePtr<Scalar>(in),
                                      NodePtr<Scalar>(std::forward<Args>(args))...);
}

}  // namespace ginn

#endif  // GINN_NODE_AFFINE_H
