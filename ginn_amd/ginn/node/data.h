// Value-holding nodes: BaseDataNode (value + gradient tensors, the base of
// almost every op node) and DataNode (a leaf holding data) with its factories.
// Mirrors ginn/node/data.h:27-114.
#ifndef GINN_NODE_DATA_H
#define GINN_NODE_DATA_H

#include <ginn/node.h>

namespace ginn {

template <typename Scalar = Real>
class BaseDataNode : public Node<Scalar> {
  Tensor<Scalar> fx_, dfx_;
  bool has_grad_ = true;
  mutable bool lazy_zero_ = false;  // dfx_ holds no value yet: see BaseNode::GradUse

 public:
  BaseDataNode(DevPtr dev, const std::vector<BaseNodePtr>& ins) : Node<Scalar>(ins), fx_(dev), dfx_(dev) {}
  BaseDataNode(DevPtr dev, const Shape& shape, const std::vector<BaseNodePtr>& ins)
      : Node<Scalar>(ins), fx_(dev, shape), dfx_(dev) {}
  // Device = the highest-precedence device among the inputs.
  template <typename NodeType>
  BaseDataNode(std::vector<NodeType> ins)
      : Node<Scalar>(std::move(ins)), fx_(best_dev(this->ins_)), dfx_(fx_.dev()) {}
  BaseDataNode(DevPtr dev = cpu()) : fx_(dev), dfx_(dev) {}
  BaseDataNode(const Shape& shape) : fx_(cpu(), shape), dfx_(cpu()) {}
  BaseDataNode(DevPtr dev, const Shape& shape) : fx_(dev, shape), dfx_(dev) {}
  BaseDataNode(const std::initializer_list<BaseNodePtr>& ins) : BaseDataNode(std::vector<BaseNodePtr>(ins)) {}
  BaseDataNode(DevPtr dev, const std::initializer_list<BaseNodePtr>& ins)
      : BaseDataNode(dev, std::vector<BaseNodePtr>(ins)) {}

  const Tensor<Scalar>& value() const override { return fx_; }
  // A gradient flagged by reset_grad_lazy() is cleared before anybody sees it.
  const Tensor<Scalar>& grad() const override {
    if (lazy_zero_) {
      lazy_zero_ = false;
      const_cast<Tensor<Scalar>&>(dfx_).set_zero();
      ++internal::lazy_grad_settles();
    }
    return dfx_;
  }
  using Node<Scalar>::value;
  using Node<Scalar>::grad;
  Tensor<Scalar>& grad_storage() override { return dfx_; }

  bool owns_grad() const override { return is_floating_point_v<Scalar>; }
  void reset_grad_lazy() override {
    if (!this->owns_grad()) {  // a view or an in-place node built on this class
      this->reset_grad();
      return;
    }
    lazy_zero_ = false;
    this->init_grad();
    lazy_zero_ = this->has_grad() && dfx_.size() > 0;
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

  std::string name() const override = 0;
};

// Inside a node whose gradient tensor is a view of the WHOLE gradient of the
// node IN (its input 0): the flag of a lazily reset gradient lives in IN.
#define GINN_GRAD_IS_VIEW_OF(IN)                                                               \
  bool owns_grad() const override { return false; }                                            \
  bool take_lazy_zero() override { return IN->take_lazy_zero(); }                              \
  bool lazy_zero() const override { return IN->lazy_zero(); }                                  \
  void clear_lazy_zero() override {}                                                           \
  BaseNode::GradUse grad_use(size_t index) const override {                                    \
    return index == 0 ? BaseNode::GradUse::Aliases : BaseNode::GradUse::Accumulates;           \
  }                                                                                            \
  const Tensor<Scalar>& grad() const override {                                                \
    if (IN->lazy_zero()) (void)std::as_const(*IN).grad();                                      \
    return BaseDataNode<Scalar>::grad();                                                       \
  }                                                                                            \
  using Node<Scalar>::grad;

// Inside a node whose grad() IS the gradient tensor of the node IN (its input 0):
// IN sizes and clears it, this node has nothing to prepare.
#define GINN_GRAD_IS_ALIAS_OF(IN)                                                              \
  void reset_grad() override {}                                                                \
  bool describe_reset_grad(std::vector<LaunchDesc>&) override { return true; }                 \
  GINN_GRAD_IS_ALIAS_OF_BUT_FOR_RESET(IN)

// The same without reset_grad() / describe_reset_grad(), for nodes that keep state of their own per pass.
#define GINN_GRAD_IS_ALIAS_OF_BUT_FOR_RESET(IN)                                                \
  void init_grad() override {}                                                                 \
  bool owns_grad() const override { return false; }                                            \
  bool take_lazy_zero() override { return IN->take_lazy_zero(); }                              \
  bool lazy_zero() const override { return IN->lazy_zero(); }                                  \
  void clear_lazy_zero() override {}                                                           \
  Tensor<Scalar>& grad_storage() override { return IN->grad_storage(); }                       \
  BaseNode::GradUse grad_use(size_t index) const override {                                    \
    return index == 0 ? BaseNode::GradUse::Aliases : BaseNode::GradUse::Accumulates;           \
  }

// A node whose value is a row of column blocks, one per part: where each part
// starts and how many columns it has, as of the last forward pass.  What
// RowwiseUncat needs to know of the node that laid the columns out
// (ginn/node/layout.h:221-315: RowwiseCatNode::offsets() / extents()).
class ColumnPartition {
 public:
  virtual ~ColumnPartition() = default;
  virtual const std::vector<Size>& offsets() const = 0;
  virtual const std::vector<Size>& extents() const = 0;
};

// Leaf node; born forwarded, reset_forwarded() does nothing.
template <typename Scalar = Real>
class DataNode : public BaseDataNode<Scalar> {
 public:
  DataNode(DevPtr dev = cpu()) : BaseDataNode<Scalar>(dev) { this->forwarded = true; }
  DataNode(Shape shape) : BaseDataNode<Scalar>(std::move(shape)) { this->forwarded = true; }
  DataNode(DevPtr dev, Shape shape) : BaseDataNode<Scalar>(std::move(dev), std::move(shape)) {
    this->forwarded = true;
  }

  using Node<Scalar>::value;
  using Node<Scalar>::grad;

  void move_to(const DevPtr& to) {
    value().move_to(to);
    grad().move_to(to);
  }
  void fill(Scalar val) { value().fill(val); }
  void set_zero() { value().set_zero(); }
  void set_ones() { value().set_ones(); }
  void set_random() { value().set_random(); }
  void reset_forwarded() override {}

  template <typename Other>
  auto cast() const {
    auto out = make_ptr<DataNode<Other>>(this->dev(), this->shape());
    out->set_has_grad(this->has_grad());
    out->forwarded = this->forwarded;
    out->value() = this->value().template cast<Other>();
    if (this->grad().size() > 0) out->grad() = this->grad().template cast<Other>();
    return out;
  }

  Shape shape() const override { return value().shape(); }
  std::string name() const override { return "DataNode"; }
};

template <typename Scalar = Real>
using DataPtr = Ptr<DataNode<Scalar>>;

// A constant with the shape its input has at forward time; no gradient flows
// through it (ginn/node/data.h:119-137).
template <typename Scalar = Real>
class ConstantLikeNode : public BaseDataNode<Scalar> {
  Scalar val_;

  void forward_() override {
    this->value().resize(this->in()->shape());
    this->value().fill(val_);
  }

 public:
  ConstantLikeNode(NodePtr<Scalar> in, Real val) : BaseDataNode<Scalar>({in}), val_(val) {}
  std::string name() const override { return "ConstantLike"; }
};

GINN_MAKE_TEMPLATE_FACTORY(Data);

template <typename Scalar = Real>
auto Data(DevPtr dev, std::initializer_list<Size> shape) {
  return Data<Scalar>(dev, Shape(shape));
}
template <typename Scalar = Real>
auto FixedData(DevPtr dev, std::initializer_list<Size> shape) {
  return FixedData<Scalar>(dev, Shape(shape));
}

template <typename Scalar = Real>
auto Constant(DevPtr dev, const Shape& shape, Scalar val) {
  auto x = FixedData<Scalar>(dev, shape);
  x->value().fill(val);
  return x;
}
template <typename Scalar = Real>
auto Zero(DevPtr dev, const Shape& s) {
  return Constant<Scalar>(dev, s, Scalar(0));
}
template <typename Scalar = Real>
auto Ones(DevPtr dev, const Shape& s) {
  return Constant<Scalar>(dev, s, Scalar(1));
}

template <typename Scalar = Real>
auto Random(DevPtr dev, const Shape& shape) {
  auto x = Data<Scalar>(dev, shape);
  x->value().set_random();
  return x;
}
template <typename Scalar = Real>
auto Random(const Shape& shape) {
  return Random<Scalar>(cpu(), shape);
}
template <typename Scalar = Real>
auto FixedRandom(DevPtr dev, const Shape& shape) {
  auto x = FixedData<Scalar>(dev, shape);
  x->value().set_random();
  return x;
}

template <typename Scalar, typename InScalar>
auto ConstantLike(NodePtr<InScalar> x, Scalar val) {
  return make_ptr<ConstantLikeNode<Scalar>>(x, val);
}
template <typename Scalar>
auto ZeroLike(NodePtr<Scalar> x) {
  return ConstantLike<Scalar>(x, Scalar(0));
}
template <typename Scalar>
auto OnesLike(NodePtr<Scalar> x) {
  return ConstantLike<Scalar>(x, Scalar(1));
}
// The derived-pointer forms that callers have in hand (Ptr<DataNode<S>> etc.).
template <typename NodeType, typename Scalar = typename NodeType::Scalar>
auto ZeroLike(const Ptr<NodeType>& x) {
  return ZeroLike<Scalar>(NodePtr<Scalar>(x));
}
template <typename NodeType, typename Scalar = typename NodeType::Scalar>
auto OnesLike(const Ptr<NodeType>& x) {
  return OnesLike<Scalar>(NodePtr<Scalar>(x));
}

// Values<2>({{1, 2, 3}, {4, 5, 6}}): a 2 x 3 data node from a literal, outermost
// list = dimension 0 (ginn/node/data.h:211-221).
template <int Rank, typename Scalar = Real>
auto Values(DevPtr dev, NestedInitList<Rank, Scalar> val) {
  auto x = Data<Scalar>(std::move(dev), shape_of<Size, Rank, Scalar>(val));
  x->value().template set<Rank>(val);
  return x;
}
template <int Rank, typename Scalar = Real>
auto Values(NestedInitList<Rank, Scalar> val) {
  return Values<Rank, Scalar>(cpu(), val);
}

// Data node with the given shape and values in storage (column-major) order.
template <typename Scalar = Real>
auto Values(DevPtr dev, const Shape& shape, const std::vector<Scalar>& vals) {
  auto x = Data<Scalar>(cpu(), shape);
  x->value().set(vals);
  x->move_to(dev);
  return x;
}

}  // namespace ginn

#endif  // GINN_NODE_DATA_H
