// Trainable parameter node (ginn/node/weight.h:29-131): the value tensor is
// shared between tied copies, the gradient is per copy; born forwarded.
#ifndef GINN_NODE_WEIGHT_H
#define GINN_NODE_WEIGHT_H

#include <atomic>
#include <mutex>

#include <ginn/node.h>

namespace ginn {

enum class Copy { Tied, Deep };

template <typename Scalar = Real>
class WeightNode : public Node<Scalar> {
  static size_t next_id() {
    static std::atomic<size_t> counter{0};
    return counter++;
  }

  size_t id_;
  Tensor<Scalar> dfx_;
  std::shared_ptr<Tensor<Scalar>> fx_;
  std::shared_ptr<std::mutex> access_;
  bool has_grad_ = true;
  mutable bool lazy_zero_ = false;  // dfx_ holds no value yet: see BaseNode::GradUse

 public:
  std::string label;

  WeightNode(DevPtr dev = cpu(), const Shape& shape = {0})
      : id_(next_id()),
        dfx_(dev),
        fx_(std::make_shared<Tensor<Scalar>>(dev, shape)),
        access_(std::make_shared<std::mutex>()) {
    this->forwarded = true;
  }
  // Deep copy: own value, own gradient, new identity.
  WeightNode(const WeightNode& other)
      : Node<Scalar>(static_cast<const Node<Scalar>&>(other)),
        id_(next_id()),
        dfx_(other.dfx_),
        fx_(std::make_shared<Tensor<Scalar>>(*other.fx_)),
        access_(std::make_shared<std::mutex>()),
        has_grad_(other.has_grad_) {}

  Tensor<Scalar>& value() {
    GINN_ASSERT(static_cast<bool>(fx_));
    return *fx_;
  }
  const Tensor<Scalar>& value() const override {
    GINN_ASSERT(static_cast<bool>(fx_));
    return *fx_;
  }
  // A gradient flagged by reset_grad_lazy() is cleared before anybody sees it.
  const Tensor<Scalar>& grad() const override {
    if (lazy_zero_) {
      lazy_zero_ = false;
      const_cast<Tensor<Scalar>&>(dfx_).set_zero();
      ++internal::lazy_grad_settles();
    }
    return dfx_;
  }
  using Node<Scalar>::grad;
  Tensor<Scalar>& grad_storage() override { return dfx_; }
  bool owns_grad() const override { return is_floating_point_v<Scalar>; }
  void reset_grad_lazy() override {
    lazy_zero_ = false;
    this->init_grad();
    lazy_zero_ = owns_grad() && has_grad_ && dfx_.size() > 0;
  }
  bool take_lazy_zero() override {
    const bool was = lazy_zero_;
    lazy_zero_ = false;
    if (was && internal::lazy_take_log()) internal::lazy_take_log()->push_back(this);
    return was;
  }
  bool lazy_zero() const override { return lazy_zero_; }
  void clear_lazy_zero() override { lazy_zero_ = false; }

  bool has_grad() const override { return has_grad_; }
  virtual void set_has_grad(bool hg) { has_grad_ = hg; }
  size_t id() const { return id_; }
  std::mutex& access() { return *access_; }
  void reset_forwarded() override {}

  void move_to(const DevPtr& to) {
    fx_->move_to(to);
    dfx_.move_to(to);
  }

  // Share value, identity and lock with `other`; the gradient stays separate.
  void tie(const Ptr<WeightNode>& other) {
    if (!other) return;
    id_ = other->id_;
    fx_ = other->fx_;
    dfx_.move_to(fx_->dev());
    dfx_ = other->dfx_;
    access_ = other->access_;
    has_grad_ = other->has_grad_;
  }

  auto copy(Copy mode = Copy::Tied) {
    if (mode == Copy::Deep) return make_ptr<WeightNode>(*this);
    auto tied = make_ptr<WeightNode>(fx_->dev());
    tied->id_ = id_;
    tied->fx_ = fx_;
    tied->dfx_ = dfx_;
    tied->access_ = access_;
    tied->has_grad_ = has_grad_;
    return tied;
  }

  template <typename Rhs>
  void fill(Rhs val) {
    value().fill(Scalar(val));
  }
  void set_zero() { value().set_zero(); }
  void set_ones() { value().set_ones(); }
  void set_random() { value().set_random(); }

  Shape shape() const override { return value().shape(); }
  std::string name() const override {
    std::string s = "Weight" + std::to_string(id_) + " (";
    const Shape sh = shape();
    for (size_t i = 0; i < sh.size(); ++i) s += (i ? "," : "") + std::to_string(sh[i]);
    return s + ")";
  }
};

template <typename Scalar>
using WeightPtr = Ptr<WeightNode<Scalar>>;

template <typename Scalar = Real>
auto Weight(DevPtr dev = cpu(), const Shape& s = {0}) {
  return make_ptr<WeightNode<Scalar>>(dev, s);
}
template <typename Scalar = Real>
auto Weight(DevPtr dev, std::initializer_list<Size> shape) {
  return Weight<Scalar>(dev, Shape(shape));
}
template <typename Scalar = Real>
auto FixedWeight(DevPtr dev = cpu(), const Shape& s = {0}) {
  auto w = Weight<Scalar>(dev, s);
  w->set_has_grad(false);
  return w;
}

}  // namespace ginn

#endif  // GINN_NODE_WEIGHT_H
