// Layout nodes used by Autobatch and by the configurations of the product
// path: Dim, Cat, RowwiseCat / RowwiseUncat, ColBroadcast, Slice, Reshape, Map
// (ginn/node/layout.h).  All are data movement on column-major storage.
#ifndef GINN_NODE_LAYOUT_H
#define GINN_NODE_LAYOUT_H

#include <ginn/cpu_ops.h>
#include <ginn/node/data.h>
#include <ginn/node/slices.h>
#include <ginn/nonlin.h>

namespace ginn {

namespace internal {
// The device type under which values of Scalar are MOVED, bit for bit: Int (indices, conditions) travels
// as 4-byte words through the copies of the 4-byte floating type.  The layout nodes below are
// instantiated and tested on Int in the reference (test/nodes.cu.cpp:66-306); their backward passes are
// floating-point only.
template <typename Scalar>
inline ginn_hip_dtype move_dtype_of() {
  if constexpr (is_floating_point_v<Scalar>) {
    return dtype_of<Scalar>();
  } else {
    static_assert(sizeof(Scalar) == 4, "only 4-byte integers are moved as words");
    return GINN_HIP_F32;
  }
}
template <typename Scalar>
void copy_2d(Tensor<Scalar>& dst, Size dst_off, Size ldd, const Tensor<Scalar>& src, Size src_off, Size lds,
             Size rows, Size cols, bool accumulate) {
  GINN_ASSERT(!accumulate || is_floating_point_v<Scalar>, "only floating-point tensors are added to");
  if (dst.dev()->kind() == CPU) {
    host::copy_2d<Scalar>(rows, cols, src.data() + src_off, lds, dst.data() + dst_off, ldd, accumulate);
    return;
  }
  require_gpu(dst.dev(), "copy_2d");
  GINN_HIP_CALL(ginn_hip_copy_2d(ctx_of(dst), move_dtype_of<Scalar>(), static_cast<int>(rows), static_cast<int>(cols),
                                 src.data() + src_off, static_cast<int>(lds), dst.data() + dst_off,
                                 static_cast<int>(ldd), accumulate ? 1 : 0));
}
// dst (+)= src over n contiguous elements, as a description for the level executor.
template <typename Scalar>
LaunchDesc copy_desc(Scalar* dst, const Scalar* src, Size n, bool accumulate) {
  LaunchDesc d;
  d.dtype = move_dtype_of<Scalar>();  // (integer nodes describe nothing: they run their copies themselves)
  d.kind = GINN_HIP_MULTI_SUM;
  d.accumulate = accumulate;
  d.n = static_cast<size_t>(n);
  d.dst = dst;
  d.src[0] = src;
  return d;
}
}  // namespace internal

// A lazily evaluated size (ginn/node/layout.h:66-112).
class DimNode : public BaseNode {
 protected:
  Size dim_ = 0;
  Size index_ = 0;
  void forward_() override {
    if (!ins().empty()) dim_ = in()->shape().at(static_cast<size_t>(index_));
  }

 public:
  DimNode() = default;
  DimNode(Size n) : dim_(n) {}
  DimNode(BaseNodePtr e, Size index) : BaseNode(std::vector<BaseNodePtr>{e}), index_(index) {}
  DevPtr dev() const override { return null_dev(); }
  bool has_grad() const override { return false; }
  Size value() { return dim_; }
  Shape shape() const override {
    GINN_THROW("Dim has no shape!");
    return {};
  }
  std::string name() const override { return "Dim"; }
};
using DimPtr = Ptr<DimNode>;
GINN_MAKE_FACTORY(Dim);

// Stacks the rank-2 folds of the inputs on top of each other (along rows).
template <typename Scalar>
class CatNode : public BaseDataNode<Scalar> {
  std::vector<NodePtr<Scalar>> ins_;

  void forward_() override {
    Size rows = 0;
    const Size cols = ins_[0]->value().cols();
    for (auto& in : ins_) {
      GINN_ASSERT(in->value().cols() == cols, "Cat: column counts differ");
      rows += in->value().rows();
    }
    value().resize(rows, cols);
    Size at = 0;
    for (auto& in : ins_) {
      const Size r = in->value().rows();
      internal::copy_2d(value(), at, rows, in->value(), 0, r, r, cols, false);
      at += r;
    }
  }
  void backward_() override {
    const Size rows = value().rows(), cols = value().cols();
    Size at = 0;
    for (auto& in : ins_) {
      const Size r = in->value().rows();
      if (in->has_grad()) internal::copy_2d(in->grad(), 0, r, grad(), at, rows, r, cols, true);
      at += r;
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  // Single-column inputs are contiguous pieces of the result.
  bool describe_forward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    Size rows = 0;
    for (auto& in : ins_) {
      if (in->value().cols() != 1) return false;
      rows += in->value().rows();
    }
    value().resize(rows, 1);
    Size at = 0;
    for (auto& in : ins_) {
      out.push_back(internal::copy_desc<Scalar>(value().data() + at, in->value().data(), in->value().rows(), false));
      at += in->value().rows();
    }
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || value().cols() != 1 || !is_floating_point_v<Scalar>) return false;
    Size at = 0;
    for (auto& in : ins_) {
      const Size r = in->value().rows();
      if (in->has_grad()) out.push_back(internal::copy_desc<Scalar>(in->grad().data(), grad().data() + at, r, true));
      at += r;
    }
    return true;
  }
  CatNode(const std::vector<NodePtr<Scalar>>& ins) : BaseDataNode<Scalar>(ins), ins_(ins) {}
  template <typename... Args>
  CatNode(const NodePtr<Scalar>& in, Args&&... args) : CatNode(std::vector<NodePtr<Scalar>>{in, args...}) {}
  std::string name() const override { return "Cat"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Cat);

// Concatenates along columns (the batch dimension of a rank-2 view) and
// remembers where each input went (ginn/node/layout.h:221-273).  Columns are
// contiguous, so every piece is one block copy.
template <typename Scalar>
class RowwiseCatNode : public BaseDataNode<Scalar>, public ColumnPartition {
  std::vector<NodePtr<Scalar>> ins_;
  std::vector<Size> offsets_, extents_;

  void forward_() override {
    const Size rows = ins_[0]->value().rows();
    Size cols = 0;
    for (auto& in : ins_) {
      GINN_ASSERT(in->value().rows() == rows, "RowwiseCat: row counts differ");
      cols += in->value().cols();
    }
    value().resize(rows, cols);
    offsets_.clear();
    extents_.clear();
    Size at = 0;
    for (auto& in : ins_) {
      const Size c = in->value().cols();
      internal::copy_2d(value(), at * rows, rows, in->value(), 0, rows, rows, c, false);
      offsets_.push_back(at);
      extents_.push_back(c);
      at += c;
    }
  }
  void backward_() override {
    const Size rows = value().rows();
    Size at = 0;
    for (auto& in : ins_) {
      const Size c = in->value().cols();
      if (in->has_grad()) internal::copy_2d(in->grad(), 0, rows, grad(), at * rows, rows, rows, c, true);
      at += c;
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  const std::vector<Size>& offsets() const override { return offsets_; }
  const std::vector<Size>& extents() const override { return extents_; }
  bool describe_forward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    const Size rows = ins_[0]->value().rows();
    Size cols = 0;
    for (auto& in : ins_) {
      GINN_ASSERT(in->value().rows() == rows, "RowwiseCat: row counts differ");
      cols += in->value().cols();
    }
    value().resize(rows, cols);
    offsets_.clear();
    extents_.clear();
    Size at = 0;
    for (auto& in : ins_) {
      const Size c = in->value().cols();
      out.push_back(internal::copy_desc<Scalar>(value().data() + at * rows, in->value().data(), rows * c, false));
      offsets_.push_back(at);
      extents_.push_back(c);
      at += c;
    }
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || !is_floating_point_v<Scalar>) return false;
    const Size rows = value().rows();
    Size at = 0;
    for (auto& in : ins_) {
      const Size c = in->value().cols();
      if (in->has_grad())
        out.push_back(internal::copy_desc<Scalar>(in->grad().data(), grad().data() + at * rows, rows * c, true));
      at += c;
    }
    return true;
  }
  RowwiseCatNode(const std::vector<NodePtr<Scalar>>& ins) : BaseDataNode<Scalar>(ins), ins_(ins) {}
  template <typename... Args>
  RowwiseCatNode(const NodePtr<Scalar>& in, Args&&... args)
      : RowwiseCatNode(std::vector<NodePtr<Scalar>>{in, args...}) {}
  std::string name() const override { return "RowwiseCat"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(RowwiseCat);

// Zero-copy view of the column range that input `index` of `cat` occupies in
// x (= something computed column-wise from cat); value and gradient both alias
// x's storage (ginn/node/layout.h:276-315).  `cat` is the node that laid the
// columns out: a RowwiseCat, or a GatherProd, which is then x itself.
template <typename Scalar>
class RowwiseUncatNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Size index_;
  BaseNodePtr cat_node_;
  const ColumnPartition* cat_;

  void forward_() override {
    const Size off = cat_->offsets().at(static_cast<size_t>(index_));
    const Size ext = cat_->extents().at(static_cast<size_t>(index_));
    const Size rows = in_->value().rows();
    value().map(in_->value(), {rows, ext}, rows * off);
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  bool has_grad() const override { return in_->has_grad(); }
  bool owns_grad() const override { return false; }  // a window of x's gradient
  void init_grad() override {
    if (!has_grad()) return;
    const Size off = cat_->offsets().at(static_cast<size_t>(index_));
    const Size ext = cat_->extents().at(static_cast<size_t>(index_));
    const Size rows = in_->value().rows();
    grad().map(in_->grad(), {rows, ext}, rows * off);
  }
  // The gradient is a window of x's gradient, which x zeroes itself.
  void reset_grad() override { init_grad(); }
  // A view has nothing to launch: mapping is all of its work in every pass.
  bool describe_forward(std::vector<LaunchDesc>&) override {
    forward_();
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>&) override { return true; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    init_grad();
    return true;
  }
  template <typename CatNode>
  RowwiseUncatNode(NodePtr<Scalar> x, Size index, Ptr<CatNode> cat)
      : BaseDataNode<Scalar>(static_cast<BaseNode*>(cat.get()) == x.get()
                                 ? std::vector<BaseNodePtr>{x}
                                 : std::vector<BaseNodePtr>{x, cat}),
        in_(x), index_(index), cat_node_(cat), cat_(cat.get()) {}
  std::string name() const override { return "RowwiseUncat"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(RowwiseUncat);

// [rows x 1] -> [rows x cols]; with cols == 1 the node aliases its input
// (ginn/node/layout.h:864-920).
template <typename Scalar>
class ColBroadcastNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  DimPtr cols_;

  void forward_() override {
    auto& x = in_->value();
    GINN_ASSERT(x.cols() == 1);
    const Size cols = cols_->value();
    if (cols > 1) {
      internal::require_gpu(this->dev(), "ColBroadcast");
      value().resize(x.rows(), cols);
      GINN_HIP_CALL(ginn_hip_col_broadcast(internal::ctx_of(x), internal::move_dtype_of<Scalar>(), static_cast<int>(x.rows()),
                                           static_cast<int>(cols), x.data(), value().data()));
    } else {
      value().map(in_->value(), in_->value().shape());
    }
  }
  void backward_() override {
    if constexpr (is_floating_point_v<Scalar>)
      if (in_->has_grad() && cols_->value() > 1)
        GINN_HIP_CALL(ginn_hip_row_sum(internal::ctx_of(grad()), dtype_of<Scalar>(), static_cast<int>(grad().rows()),
                                     static_cast<int>(grad().cols()), grad().data(), in_->grad().data(), 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  ColBroadcastNode(NodePtr<Scalar> in, DimPtr cols)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{in, cols}), in_(in), cols_(cols) {}
  ColBroadcastNode(NodePtr<Scalar> in, Size cols) : ColBroadcastNode(in, make_ptr<DimNode>(cols)) {}

  bool has_grad() const override {
    if (cols_->value() == 1) return in_->has_grad();
    return BaseDataNode<Scalar>::has_grad();
  }
  bool owns_grad() const override { return false; }  // with one column the gradient is the input's
  void init_grad() override {
    if (!has_grad()) return;
    if (cols_->value() > 1) {
      if (grad().shape() != value().shape()) grad().resize(value().shape());
    } else {
      grad().map(in_->grad(), in_->grad().shape());
    }
  }
  void reset_grad() override {
    init_grad();
    // An aliased gradient is zeroed by the input itself.
    if (has_grad() && cols_->value() > 1) grad().set_zero();
  }
  // With one column the node is a view (nothing to launch); the broadcast
  // proper and its row sums run as usual.
  bool describe_forward(std::vector<LaunchDesc>&) override {
    if (cols_->value() > 1) return false;
    forward_();
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>&) override { return cols_->value() == 1; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    if (cols_->value() > 1) return false;
    init_grad();
    return true;
  }
  std::string name() const override { return "ColBroadcast"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(ColBroadcast);

// Rectangular window of the rank-2 fold: rows [r0, r0 + nr), columns
// [c0, c0 + nc) (the rank <= 2 case of ginn/node/layout.h:563-629).
template <typename Scalar>
class SliceNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Shape offsets_, sizes_;

  void window(Size& r0, Size& c0, Size& nr, Size& nc) const {
    r0 = offsets_[0];
    nr = sizes_[0];
    c0 = offsets_.size() > 1 ? offsets_[1] : 0;
    nc = sizes_.size() > 1 ? sizes_[1] : in_->value().cols();
  }
  void forward_() override {
    GINN_ASSERT(sizes_.size() <= 2, "Slice: only rank 1 and 2 windows are part of this build");
    Size r0, c0, nr, nc;
    window(r0, c0, nr, nc);
    const Size rows = in_->value().rows();
    GINN_ASSERT(r0 + nr <= rows && c0 + nc <= in_->value().cols(), "Slice: window out of range");
    if (sizes_.size() > 1) value().resize(sizes_);
    else value().resize(nr, nc);
    internal::copy_2d(value(), 0, nr, in_->value(), c0 * rows + r0, rows, nr, nc, false);
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    Size r0, c0, nr, nc;
    window(r0, c0, nr, nc);
    const Size rows = in_->value().rows();
    internal::copy_2d(in_->grad(), c0 * rows + r0, rows, grad(), 0, nr, nr, nc, true);
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  // A window of whole columns, or inside a single column, is contiguous.
  bool contiguous(Size nr, Size nc) const { return nc == 1 || nr == in_->value().rows(); }
  bool describe_forward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || sizes_.size() > 2 || !is_floating_point_v<Scalar>) return false;
    Size r0, c0, nr, nc;
    window(r0, c0, nr, nc);
    const Size rows = in_->value().rows();
    if (!contiguous(nr, nc)) return false;
    GINN_ASSERT(r0 + nr <= rows && c0 + nc <= in_->value().cols(), "Slice: window out of range");
    if (sizes_.size() > 1) value().resize(sizes_);
    else value().resize(nr, nc);
    out.push_back(internal::copy_desc<Scalar>(value().data(), in_->value().data() + c0 * rows + r0, nr * nc, false));
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>& out) override {
    if (value().dev()->kind() != GPU || sizes_.size() > 2 || !is_floating_point_v<Scalar>) return false;
    Size r0, c0, nr, nc;
    window(r0, c0, nr, nc);
    if (!contiguous(nr, nc)) return false;
    const Size rows = in_->value().rows();
    if (in_->has_grad())
      out.push_back(internal::copy_desc<Scalar>(in_->grad().data() + c0 * rows + r0, grad().data(), nr * nc, true));
    return true;
  }
  SliceNode(const NodePtr<Scalar>& x, Shape offsets, Shape sizes)
      : BaseDataNode<Scalar>({x}), in_(x), offsets_(std::move(offsets)), sizes_(std::move(sizes)) {
    GINN_ASSERT(offsets_.size() == sizes_.size());
    GINN_ASSERT(!sizes_.empty());
  }
  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() == 1);
    BaseNode::ins_ = ins;
    in_ = dynamic_ptr_cast<Node<Scalar>>(ins.front());
  }
  std::string name() const override { return "Slice"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Slice);

// Same storage, another shape (ginn/node/layout.h:472-521).
template <typename Scalar>
class ReshapeNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Shape shape_;

  void forward_() override { value().map(in_->value(), shape_); }

 public:
  using BaseDataNode<Scalar>::value;
  GINN_GRAD_IS_VIEW_OF(in_)
  bool has_grad() const override { return in_->has_grad(); }
  void init_grad() override {
    if (has_grad()) this->grad_storage().map(in_->grad_storage(), shape_);
  }
  void reset_grad() override { init_grad(); }
  // A view has nothing to launch: mapping is all of its work in every pass.
  bool describe_forward(std::vector<LaunchDesc>&) override {
    forward_();
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>&) override { return true; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    init_grad();
    return true;
  }
  ReshapeNode(const NodePtr<Scalar>& x, Shape shape) : BaseDataNode<Scalar>({x}), in_(x), shape_(std::move(shape)) {}
  std::string name() const override { return "Reshape"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Reshape);

// The input under the shape that Tensor::reduce gives it for `rank` axes: trailing axes folded into the
// last one kept, or axes of extent 1 appended (ginn/node/layout.h:529-561).  A view, like Reshape.
template <typename Scalar>
class RankViewNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Size rank_;

  Shape view_shape() const { return Tensor<Scalar>::reduce(in_->shape(), rank_); }
  void forward_() override { value().map(in_->value(), view_shape()); }

 public:
  using BaseDataNode<Scalar>::value;
  GINN_GRAD_IS_VIEW_OF(in_)
  bool has_grad() const override { return in_->has_grad(); }
  void init_grad() override {
    if (has_grad()) this->grad_storage().map(in_->grad_storage(), view_shape());
  }
  void reset_grad() override { init_grad(); }
  bool describe_forward(std::vector<LaunchDesc>&) override {
    forward_();
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>&) override { return true; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    init_grad();
    return true;
  }
  RankViewNode(const NodePtr<Scalar>& x, Size rank) : BaseDataNode<Scalar>({x}), in_(x), rank_(rank) {
    GINN_ASSERT(rank >= 1, "RankView: rank 0 is not handled (nor in ginn/node/layout.h:530)");
  }
  std::string name() const override { return "RankView"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(RankView);

// Identity view whose input can be rewired (ginn/node/layout.h:698-721); gives
// Autobatch a consumer for nodes that otherwise end in non-rewirable users.
template <typename Scalar>
class MapNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  void forward_() override { value().map(in_->value()); }

 public:
  using BaseDataNode<Scalar>::value;
  GINN_GRAD_IS_VIEW_OF(in_)
  bool has_grad() const override { return in_->has_grad(); }
  void init_grad() override {
    if (has_grad()) this->grad_storage().map(in_->grad_storage());
  }
  void reset_grad() override { init_grad(); }
  // A view has nothing to launch: mapping is all of its work in every pass.
  bool describe_forward(std::vector<LaunchDesc>&) override {
    forward_();
    return true;
  }
  bool describe_backward(std::vector<LaunchDesc>&) override { return true; }
  bool describe_reset_grad(std::vector<LaunchDesc>&) override {
    init_grad();
    return true;
  }
  MapNode(const NodePtr<Scalar>& x) : BaseDataNode<Scalar>({x}), in_(x) {}
  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() == 1);
    BaseNode::ins_ = ins;
    in_ = dynamic_ptr_cast<Node<Scalar>>(ins.front());
  }
  std::string name() const override { return "Map"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Map);

// Axis permutation: result extent k is the input's extent indices[k]
// (ginn/node/layout.h:723-821); backward adds the inversely permuted gradient.
// On the HIP device the copy is postponed until the value is read when the
// result's slices are matrices inside the input's memory (node/slices.h): a
// BatchedProd that multiplies them takes them from there (and puts the gradient
// there), and a BatchedProd in front whose product is still pending writes its
// result permuted; every other reader gets the copy as usual.
template <typename Scalar>
class PermuteNode : public BaseDataNode<Scalar>, public internal::SliceProvider<Scalar>, public PostponedValue {
 protected:
  NodePtr<Scalar> in_;
  Shape indices_;
  bool overwrite_ = false;  // set by InPlacePermuteNode: results replace, through a temporary
  mutable bool pending_ = false;  // forward() has run, the copy has not
  bool skip_backward_ = false;    // the only user has put the gradient into the input's already

  static Shape permute(const Shape& s, const Shape& perm) {
    Shape out(s.size());
    for (size_t i = 0; i < s.size(); ++i) out[i] = s[static_cast<size_t>(perm[i])];
    return out;
  }
  static Shape inverse(const Shape& perm) {
    Shape inv(perm.size());
    for (size_t i = 0; i < perm.size(); ++i) inv[static_cast<size_t>(perm[i])] = static_cast<Size>(i);
    return inv;
  }
  void check_permutation(const Shape& s) const {
    GINN_ASSERT(indices_.size() == s.size());
    Shape seen(s.size(), 0);
    for (Size i : indices_)
      GINN_ASSERT(i >= 0 && i < static_cast<Size>(s.size()) && !seen[static_cast<size_t>(i)]++,
                  "Indices are not a proper permutation in Permute!");
  }

  static void run(const Tensor<Scalar>& src, const Shape& src_shape, const Shape& perm, Tensor<Scalar>& dst,
                  bool accumulate) {
    if (dst.dev()->kind() == CPU) {
      if constexpr (is_floating_point_v<Scalar>)
        return host::permute<Scalar>(src_shape, perm, src.data(), dst.data(), accumulate);
    }
    internal::require_gpu(dst.dev(), "Permute");
    std::vector<long long> dims(src_shape.begin(), src_shape.end());
    std::vector<int> p(perm.begin(), perm.end());
    if constexpr (!is_floating_point_v<Scalar>) GINN_ASSERT(!accumulate, "integers are moved, not summed");
    GINN_HIP_CALL(ginn_hip_permute(internal::ctx_of(dst), internal::move_dtype_of<Scalar>(),
                                   static_cast<int>(dims.size()), dims.data(), p.data(), src.data(), dst.data(),
                                   accumulate ? 1 : 0));
  }
  Tensor<Scalar>& raw_value() const { return const_cast<Tensor<Scalar>&>(BaseDataNode<Scalar>::value()); }
  internal::SliceTaker<Scalar>* pending_product() const {
    auto* t = dynamic_cast<internal::SliceTaker<Scalar>*>(in_.get());
    return t && t->product_pending() ? t : nullptr;
  }
  // The result's slices as matrices inside `stored`, which holds the input (forward: its value) or has the
  // input's shape (backward: its gradient).
  bool slices_in_input(Scalar* stored, internal::BatchView<Scalar>& v) const {
    return internal::permuted_slices(stored, in_->shape(), indices_, v);
  }
  // The input's slices as matrices inside `stored`, which has the result's shape.
  bool slices_in_result(Tensor<Scalar>& stored, internal::BatchView<Scalar>& v) const {
    return internal::permuted_slices(stored.data(), stored.shape(), inverse(indices_), v);
  }
  void copy_now() const {
    if (auto* t = pending_product()) {  // the product in front writes its slices where the copy would put them
      internal::BatchView<Scalar> v;
      if (slices_in_result(raw_value(), v)) {
        t->produce_into(v);
        return;
      }
    }
    run(in_->value(), in_->shape(), indices_, raw_value(), false);
  }
  void forward_() override {
    const Shape s = in_->shape();
    check_permutation(s);
    raw_value().resize(permute(s, indices_));
    internal::BatchView<Scalar> v;
    const bool on_gpu = this->dev()->kind() == GPU;
    if (on_gpu && !overwrite_ && is_floating_point_v<Scalar> && raw_value().size() > 0 &&
        (internal::permuted_slices(static_cast<Scalar*>(nullptr), s, indices_, v) ||
         (pending_product() && slices_in_result(raw_value(), v)))) {
      pending_ = true;
      return;
    }
    pending_ = false;
    copy_now();
  }
  void backward_() override {
    if (skip_backward_) {
      skip_backward_ = false;
      return;
    }
    if (!in_->has_grad() || !is_floating_point_v<Scalar>) return;  // (integers carry no gradient)
    if (overwrite_) {
      // grad() is in's gradient storage under the permuted shape: permute into a
      // temporary and copy back (the reference's `.eval()`, ginn/node/layout.h:766-770).
      Tensor<Scalar> tmp(grad().dev(), in_->shape());
      run(grad(), grad().shape(), inverse(indices_), tmp, false);
      Tensor<Scalar> flat;
      flat.map(in_->grad(), in_->shape());
      flat = tmp;
    } else {
      const bool fresh = in_->take_lazy_zero();
      // The only user of a batched product's gradient: the product reads it from here, permuted.
      if (fresh)
        if (auto* t = dynamic_cast<internal::SliceTaker<Scalar>*>(in_.get())) {
          internal::BatchView<Scalar> v;
          if (slices_in_result(grad(), v) && t->take_grad_slices(v)) return;
        }
      run(grad(), grad().shape(), inverse(indices_), in_->grad(), !fresh);
    }
  }

 public:
  const Tensor<Scalar>& value() const override {
    if (pending_) {
      pending_ = false;
      copy_now();
    }
    return BaseDataNode<Scalar>::value();
  }
  using Node<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  void settle_value() override { (void)std::as_const(*this).value(); }
  Shape shape() const override { return BaseDataNode<Scalar>::value().shape(); }
  DevPtr dev() const override { return BaseDataNode<Scalar>::value().dev(); }
  BaseNode::GradUse grad_use(size_t) const override {
    return overwrite_ ? BaseNode::GradUse::Accumulates : BaseNode::GradUse::Overwrites;
  }
  bool value_slices(internal::BatchView<Scalar>& v) override {
    if (!pending_ || pending_product()) return false;
    return slices_in_input(in_->value().data(), v);
  }
  bool grad_slices(internal::BatchView<Scalar>& v, bool& accumulate) override {
    if (overwrite_ || !in_->has_grad() || this->dev()->kind() != GPU) return false;
    internal::BatchView<Scalar> probe;
    if (!internal::permuted_slices(static_cast<Scalar*>(nullptr), in_->shape(), indices_, probe)) return false;
    const bool fresh = in_->take_lazy_zero();  // before grad(): a flagged gradient would be cleared on sight
    slices_in_input(in_->grad().data(), v);
    accumulate = !fresh;
    skip_backward_ = true;
    return true;
  }
  PermuteNode(const NodePtr<Scalar>& in, Shape indices)
      : BaseDataNode<Scalar>({in}), in_(in), indices_(std::move(indices)) {}
  std::string name() const override { return "Permute"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Permute);

template <typename NodePtrType>
auto Permute(NodePtrType x, std::initializer_list<Size> indices) {
  return Permute(std::move(x), Shape(indices));
}

// Swaps two axes (ginn/node/layout.h:822-828).
template <typename NodePtrType>
auto Transpose(NodePtrType x, Size i, Size j) {
  Shape indices(x->shape().size());
  std::iota(indices.begin(), indices.end(), Size(0));
  std::swap(indices.at(static_cast<size_t>(i)), indices.at(static_cast<size_t>(j)));
  return Permute(std::move(x), std::move(indices));
}

// The sub-tensor at position `offset` of axis `dim`; the result has one axis
// less (ginn/node/layout.h:631-697).  With the input viewed as
// [inner, extent(dim), outer] this is a strided copy.
template <typename Scalar>
class ChipNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  Size offset_, dim_;

  void geometry(Size& inner, Size& extent, Size& outer) const {
    const Shape s = in_->shape();
    inner = outer = 1;
    for (Size a = 0; a < dim_; ++a) inner *= s[static_cast<size_t>(a)];
    extent = s[static_cast<size_t>(dim_)];
    for (size_t a = static_cast<size_t>(dim_) + 1; a < s.size(); ++a) outer *= s[a];
  }
  void forward_() override {
    const Shape in_s = in_->shape();
    GINN_ASSERT(dim_ >= 0 && static_cast<size_t>(dim_) < in_s.size());
    GINN_ASSERT(offset_ >= 0 && offset_ < in_s[static_cast<size_t>(dim_)]);
    GINN_ASSERT(in_s.size() >= 2 && in_s.size() <= 8, "Unexpected input rank in Chip!");
    Shape s = in_s;
    s.erase(s.begin() + dim_);
    value().resize(s);
    Size inner, extent, outer;
    geometry(inner, extent, outer);
    internal::copy_2d(value(), 0, inner, in_->value(), offset_ * inner, inner * extent, inner, outer, false);
  }
  void backward_() override {
    if (!in_->has_grad()) return;
    if constexpr (is_floating_point_v<Scalar>) {
      Size inner, extent, outer;
      geometry(inner, extent, outer);
      internal::copy_2d(in_->grad(), offset_ * inner, inner * extent, grad(), 0, inner, inner, outer, true);
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  ChipNode(const NodePtr<Scalar>& x, Size offset, Size dim) : BaseDataNode<Scalar>({x}), in_(x), offset_(offset), dim_(dim) {}
  std::string name() const override { return "Chip"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(Chip);

// An m x n grid of equally shaped tensors as one tensor of shape
// (their shape) + {m, n}: embedding lookups stacked into a batch
// (ginn/node/layout.h:350-466).  One gather kernel over a device table of the
// inputs' addresses; backward adds atomically, because a grid may hold one
// node in several places.
template <typename Scalar>
class StackNode : public BaseDataNode<Scalar> {
  std::vector<std::vector<NodePtr<Scalar>>> nodes_;
  Tensor<void*> table_;  // device copy of the address table of the pass under way

  static std::vector<BaseNodePtr> flatten(const std::vector<std::vector<NodePtr<Scalar>>>& nodes) {
    std::vector<BaseNodePtr> flat;
    for (auto& inner : nodes)
      for (auto& x : inner) flat.push_back(x);
    return flat;
  }
  // Entry j * m + i names what nodes_[i][j] yields through `get` (NULL allowed).
  template <typename Get>
  void* upload_table(Get get) {
    const size_t m = nodes_.size(), n = nodes_[0].size();
    std::vector<void*> host(m * n);
    for (size_t i = 0; i < m; ++i)
      for (size_t j = 0; j < n; ++j) host[j * m + i] = get(nodes_[i][j]);
    table_.move_to(this->dev());
    table_.resize({static_cast<Size>(host.size())});
    table_.set(host);
    return table_.data();
  }
  void forward_() override {
    internal::require_gpu(this->dev(), "Stack");
    const Size m = static_cast<Size>(nodes_.size()), n = static_cast<Size>(nodes_[0].size());
    const Shape s = nodes_[0][0]->shape();
    for (auto& inner : nodes_)
      for (auto& x : inner) GINN_ASSERT(x->shape() == s, "Input shapes mismatch!");
    Shape ns = s;
    ns.push_back(m);
    ns.push_back(n);
    value().resize(ns);
    const size_t sz = static_cast<size_t>(nodes_[0][0]->size());
    void* table = upload_table([](const NodePtr<Scalar>& x) { return static_cast<void*>(x->value().data()); });
    GINN_HIP_CALL(ginn_hip_stack(internal::ctx_of(value()), static_cast<int>(sizeof(Scalar)), sz,
                                 static_cast<size_t>(m * n), static_cast<const void* const*>(table), value().data()));
  }
  void backward_() override {
    if constexpr (is_floating_point_v<Scalar>) {
      const size_t sz = static_cast<size_t>(nodes_[0][0]->size());
      void* table = upload_table([](const NodePtr<Scalar>& x) {
        return x->has_grad() ? static_cast<void*>(x->grad().data()) : nullptr;
      });
      GINN_HIP_CALL(ginn_hip_stack_bwd(internal::ctx_of(grad()), dtype_of<Scalar>(), sz,
                                       nodes_.size() * nodes_[0].size(), static_cast<void* const*>(table),
                                       grad().data()));
    }
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  StackNode(const std::vector<std::vector<NodePtr<Scalar>>>& nodes)
      : BaseDataNode<Scalar>(flatten(nodes)), nodes_(nodes) {
    GINN_ASSERT(!nodes_.empty(), "Empty input to Stack!");
    GINN_ASSERT(!nodes_.front().empty(), "Empty input to Stack!");
    for (auto& inner : nodes_) GINN_ASSERT(inner.size() == nodes_.front().size(), "Inner container sizes mismatch!");
  }
  std::string name() const override { return "Stack"; }
};
template <typename Scalar>
auto Stack(const std::vector<std::vector<NodePtr<Scalar>>>& ins) {
  return make_ptr<StackNode<Scalar>>(ins);
}

// A [1 x cols] row repeated `rows` times; backward sums the gradient over the
// rows (ginn/node/layout.h:831-862).
template <typename Scalar>
class RowBroadcastNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> in_;
  DimPtr rows_;

  void forward_() override {
    internal::require_gpu(this->dev(), "RowBroadcast");
    auto& x = in_->value();
    GINN_ASSERT(x.shape().size() == 2);
    GINN_ASSERT(x.rows() == 1);
    const Size rows = rows_->value();
    value().resize(rows, x.cols());
    GINN_HIP_CALL(ginn_hip_row_broadcast(internal::ctx_of(x), internal::move_dtype_of<Scalar>(), static_cast<int>(rows),
                                         static_cast<int>(x.cols()), x.data(), value().data()));
  }
  void backward_() override {
    if constexpr (is_floating_point_v<Scalar>)
      if (in_->has_grad())
        GINN_HIP_CALL(ginn_hip_col_sum(internal::ctx_of(grad()), dtype_of<Scalar>(), static_cast<int>(grad().rows()),
                                     static_cast<int>(grad().cols()), grad().data(), in_->grad().data(), 1));
  }

 public:
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;
  RowBroadcastNode(const NodePtr<Scalar>& in, DimPtr rows)
      : BaseDataNode<Scalar>(std::vector<BaseNodePtr>{in, rows}), in_(in), rows_(rows) {}
  RowBroadcastNode(const NodePtr<Scalar>& in, Size rows) : RowBroadcastNode(in, make_ptr<DimNode>(rows)) {}
  std::string name() const override { return "RowBroadcast"; }
};
GINN_MAKE_SCALAR_FORWARDING_FACTORY(RowBroadcast);

// Square matrix of ones on and above the diagonal, zeros below: the causal
// attention mask (ginn/node/layout.h:922-955).  Carries no gradient.
template <typename Scalar = Real>
class UpperTriNode : public BaseDataNode<Scalar> {
  DimPtr size_;

  void forward_() override {
    const Size s = size_->value();
    value().resize(s, s);
    if (this->dev()->kind() == CPU) {
      for (Size c = 0; c < s; ++c)
        for (Size r = 0; r < s; ++r) value().data()[c * s + r] = Scalar(r <= c ? 1.f : 0.f);
      return;
    }
    internal::require_gpu(this->dev(), "UpperTri");
    GINN_HIP_CALL(ginn_hip_upper_tri(internal::ctx_of(value()), arith_dtype_of<Scalar>(), static_cast<int>(s),
                                     value().data()));
  }

 public:
  using BaseDataNode<Scalar>::value;
  bool has_grad() const override { return false; }
  UpperTriNode(DevPtr dev, DimPtr size) : BaseDataNode<Scalar>(dev, {BaseNodePtr(size)}), size_(size) {}
  UpperTriNode(DevPtr dev, Size size) : UpperTriNode(dev, Dim(size)) {}
  std::string name() const override { return "UpperTri"; }
};
GINN_MAKE_TEMPLATE_FACTORY(UpperTri);

}  // namespace ginn

#endif  // GINN_NODE_LAYOUT_H
