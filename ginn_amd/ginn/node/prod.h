// Matrix-product nodes (ginn/node/prod.h:22-187).
#ifndef GINN_NODE_PROD_H
#define GINN_NODE_PROD_H

#include <algorithm>
#include <atomic>

#include <ginn/node/data.h>
#include <ginn/node/slices.h>
#include <ginn/nonlin.h>
#include <ginn/prod.h>

namespace ginn {

// Y = A * B on the rank-2 folds; the output is always rank 2.
// Backward: dB += A^T dY, dA += dY B^T, each only if the input has a gradient.
template <typename Scalar>
class ProdNode : public BaseDataNode<Scalar> {
  NodePtr<Scalar> a_, b_;

  void forward_() override {
    value().resize(a_->value().rows(), b_->value().cols());
    if (dev()->kind() == CPU) {
      internal::cpu_prod(value(), a_->value(), b_->value());
      return;
    }
    internal::require_gpu(dev(), "Prod");
    internal::gpu_prod(value(), a_->value(), b_->value());
  }
  void backward_() override {
    using namespace internal;
    if (dev()->kind() == CPU) {  // ginn/node/prod.h:39-58
      if (b_->has_grad())
        cpu_prod(b_->grad(), a_->value(), grad(), b_->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::First);
      if (a_->has_grad())
        cpu_prod(a_->grad(), grad(), b_->value(), a_->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::Second);
      return;
    }
    // A gradient that is a leaf's (a weight's) is formed beside the pass, the other one first.
    const double flops = 2.0 * static_cast<double>(grad().size()) * static_cast<double>(a_->value().cols());
    for (const bool leaves : {false, true}) {
      if (b_->has_grad() && b_->inputs().empty() == leaves) {
        const bool fresh = b_->take_lazy_zero();
        ginn_hip_ctx* where = BesidePass::ctx_for(*b_, dev(), flops);
        gpu_prod(where, b_->grad(), a_->value(), grad(), fresh ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::First);
      }
      if (a_->has_grad() && a_->inputs().empty() == leaves) {
        const bool fresh = a_->take_lazy_zero();
        ginn_hip_ctx* where = BesidePass::ctx_for(*a_, dev(), flops);
        gpu_prod(where, a_->grad(), grad(), b_->value(), fresh ? ProdResult::Assign : ProdResult::Add,
                 ProdTranspose::Second);
      }
    }
  }

 public:
  using BaseDataNode<Scalar>::dev;
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;

  ProdNode(const NodePtr<Scalar>& a, const NodePtr<Scalar>& b) : BaseDataNode<Scalar>({a, b}), a_(a), b_(b) {}
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }

  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() == 2);
    BaseNode::ins_ = ins;
    a_ = dynamic_ptr_cast<Node<Scalar>>(ins[0]);
    b_ = dynamic_ptr_cast<Node<Scalar>>(ins[1]);
  }
  std::string name() const override { return "Prod"; }
};

GINN_MAKE_SCALAR_FORWARDING_FACTORY(Prod);

namespace internal {

// A device array of column addresses that follows a host copy: uploaded only
// when the addresses differ from those of the last call, so a graph that is
// run again with its tensors in place uploads nothing.
class ColumnTable {
  DevPtr dev_;
  void* dev_table_ = nullptr;
  size_t capacity_ = 0;
  std::vector<const void*> host_, next_;
  bool aligned_ = true;

 public:
  ColumnTable() = default;
  ColumnTable(const ColumnTable&) = delete;
  ColumnTable& operator=(const ColumnTable&) = delete;
  ~ColumnTable() {
    try {
      if (dev_table_) dev_->free(dev_table_);
    } catch (...) {  // teardown never throws
    }
  }
  void begin() {
    next_.clear();
    aligned_ = true;
  }
  // `cols` columns of `stride_bytes` each, starting at base.
  void add(const void* base, Size cols, size_t stride_bytes) {
    const char* p = static_cast<const char*>(base);
    for (Size j = 0; j < cols; ++j) next_.push_back(p + static_cast<size_t>(j) * stride_bytes);
    if (reinterpret_cast<uintptr_t>(base) % 16 != 0 || (cols > 1 && stride_bytes % 16 != 0)) aligned_ = false;
  }
  size_t size() const { return next_.size(); }
  bool aligned() const { return aligned_; }
  // The device table holding what was added since begin().
  void* commit(const DevPtr& dev, ginn_hip_ctx* ctx) {
    if (next_ == host_ && dev_table_ && dev_ == dev) return dev_table_;
    if (dev_table_ && (dev_ != dev || next_.size() > capacity_)) {
      dev_->free(dev_table_);
      dev_table_ = nullptr;
    }
    if (!dev_table_) {
      dev_ = dev;
      capacity_ = next_.size();
      dev_table_ = dev_->alloc(capacity_ * sizeof(void*));
    }
    GINN_HIP_CALL(ginn_hip_memcpy_h2d(ctx, dev_table_, next_.data(), next_.size() * sizeof(void*)));
    GINN_HIP_CALL(ginn_hip_sync(ctx));  // next_ is reused by the next call
    host_ = next_;
    return dev_table_;
  }
};

// The gradient of a left operand that many merged products share (the weight
// matrix of a recurrent cell: one merged product per time step, each adding
// dY_t X_t^T, ginn/node/prod.h:57-63).  Nothing reads a leaf's gradient before
// the backward pass ends, so while a pass is running (FoldWindow) the products
// only list their columns here and the end of the pass runs ONE product that
// sums over the columns of all of them (ginn_hip_gemm_outer_sum).  The tables
// belong to the node that queued first; in a graph that is run again with its
// tensors in place they are the same every pass and nothing is uploaded.
struct LateOuterSum {
  void* target;
  ginn_hip_ctx* ctx;
  DevPtr dev;
  ginn_hip_dtype dtype;
  Size m, n;
  float beta;
  ColumnTable* a_cols;
  ColumnTable* b_cols;
};
inline std::vector<LateOuterSum>& late_outer_sums() {
  thread_local std::vector<LateOuterSum> jobs;
  return jobs;
}
// Columns summed by postponed products so far (process-wide, for tests).
inline std::atomic<size_t>& late_outer_sum_columns() {
  static std::atomic<size_t> n{0};
  return n;
}
inline void run_late_outer_sums(int run) {
  std::vector<LateOuterSum> jobs;
  jobs.swap(late_outer_sums());
  if (!run) return;
  for (LateOuterSum& j : jobs) {
    const size_t k = j.a_cols->size();
    GINN_ASSERT(k == j.b_cols->size());
    const int aligned = j.a_cols->aligned() && j.b_cols->aligned();
    auto* ta = static_cast<const void* const*>(j.a_cols->commit(j.dev, j.ctx));
    auto* tb = static_cast<const void* const*>(j.b_cols->commit(j.dev, j.ctx));
    GINN_HIP_CALL(ginn_hip_gemm_outer_sum(j.ctx, j.dtype, static_cast<int>(j.m), static_cast<int>(j.n),
                                          static_cast<int>(k), ta, tb, j.beta, j.target, static_cast<int>(j.m),
                                          aligned));
    late_outer_sum_columns() += k;
  }
}

}  // namespace internal

// Y = A * [B_0 B_1 ... ]: the product Autobatch forms from products that share
// their left operand (ginn/autobatch.h:149-183), reading every B_i where it
// is instead of a RowwiseCat copy of them (ginn/node/layout.h:221-315); the
// reference lists this as the way to go (ginn/autobatch.h:30-38).  The value
// is one [rows(A) x sum of cols(B_i)] matrix whose column blocks RowwiseUncat
// hands out as views.  Backward: dA += dY [B_0 B_1 ...]^T as one product that
// sums over all gathered columns, dB_i += A^T dY_i written straight into the
// B_i's gradients by one product.
template <typename Scalar>
class GatherProdNode : public BaseDataNode<Scalar>, public ColumnPartition {
  NodePtr<Scalar> a_;
  std::vector<NodePtr<Scalar>> bs_;
  std::vector<Size> offsets_, extents_;
  internal::ColumnTable values_, grads_;
  internal::ColumnTable sum_a_, sum_b_;  // of the left operand's postponed gradient, when this node queued first

  // Lists dY's and the right operands' columns for the product that forms the
  // left operand's gradient at the end of the pass; false: form it now.
  bool postpone_left_gradient(ginn_hip_ctx* ctx, Size m, Size k, Size total) {
    using namespace internal;
    if (!FoldWindow::open() || !a_->inputs().empty()) return false;
    auto& jobs = late_outer_sums();
    void* target = nullptr;
    LateOuterSum* job = nullptr;
    for (auto& j : jobs)
      if (j.target == a_->grad_storage().data()) job = &j;
    if (job) {
      if (job->ctx != ctx || job->dtype != dtype_of<Scalar>() || job->m != m || job->n != k || job->dev != dev())
        return false;
    } else {
      const bool fresh = a_->take_lazy_zero();
      target = a_->grad().data();
      sum_a_.begin();
      sum_b_.begin();
      jobs.push_back({target, ctx, dev(), dtype_of<Scalar>(), m, k, fresh ? 0.f : 1.f, &sum_a_, &sum_b_});
      job = &jobs.back();
      FoldWindow::at_close(&run_late_outer_sums);
    }
    job->a_cols->add(grad().data(), total, static_cast<size_t>(m) * sizeof(Scalar));
    for (auto& b : bs_) job->b_cols->add(b->value().data(), b->value().cols(), static_cast<size_t>(k) * sizeof(Scalar));
    return true;
  }

  void forward_() override {
    internal::require_gpu(dev(), "GatherProd");
    const auto& a = a_->value();
    const Size m = a.rows(), k = a.cols();
    offsets_.clear();
    extents_.clear();
    values_.begin();
    Size total = 0;
    for (auto& b : bs_) {
      const auto& v = b->value();
      GINN_ASSERT(v.rows() == k, "GatherProd: a right operand's rows differ from the left operand's columns");
      offsets_.push_back(total);
      extents_.push_back(v.cols());
      values_.add(v.data(), v.cols(), static_cast<size_t>(k) * sizeof(Scalar));
      total += v.cols();
    }
    value().resize(m, total);
    if (m == 0 || total == 0) return;
    ginn_hip_ctx* ctx = internal::ctx_of(value());
    auto* table = static_cast<const void* const*>(values_.commit(dev(), ctx));
    GINN_HIP_CALL(ginn_hip_gemm_gathered(ctx, dtype_of<Scalar>(), internal::OP_N, internal::OP_N,
                                         static_cast<int>(m), static_cast<int>(total), static_cast<int>(k),
                                         a.data(), static_cast<int>(m), nullptr, 0, table, 0.f, value().data(),
                                         static_cast<int>(m), nullptr, values_.aligned()));
  }

  void backward_() override {
    const auto& a = a_->value();
    const Size m = a.rows(), k = a.cols(), total = value().cols();
    if (m == 0 || total == 0 || k == 0) return;
    ginn_hip_ctx* ctx = internal::ctx_of(value());
    if (a_->has_grad() && !postpone_left_gradient(ctx, m, k, total)) {
      // dA[m x k] += dY[m x total] * X^T, X's columns gathered: they are the
      // stored columns of the transposed operand, indexed along the sum.
      auto* table = static_cast<const void* const*>(values_.commit(dev(), ctx));
      const bool fresh = a_->take_lazy_zero();
      GINN_HIP_CALL(ginn_hip_gemm_gathered(ctx, dtype_of<Scalar>(), internal::OP_N, internal::OP_T,
                                           static_cast<int>(m), static_cast<int>(k), static_cast<int>(total),
                                           grad().data(), static_cast<int>(m), nullptr, 0, table,
                                           fresh ? 0.f : 1.f, a_->grad().data(), static_cast<int>(m), nullptr,
                                           values_.aligned()));
    }
    size_t with_grad = 0;
    for (auto& b : bs_) with_grad += b->has_grad() ? 1 : 0;
    // One launch adds into every gradient at once, which is only right when no
    // two of them are the same memory (a node that is the right operand of two
    // merged products appears twice).
    bool distinct = true;
    if (with_grad == bs_.size()) {
      std::vector<const void*> bases;
      for (auto& b : bs_)
        if (b->value().cols() > 0) bases.push_back(b->grad().data());
      std::sort(bases.begin(), bases.end());
      distinct = std::adjacent_find(bases.begin(), bases.end()) == bases.end();
    }
    if (with_grad == bs_.size() && distinct) {
      // dB_i[k x n_i] += A^T * dY[:, block i] for all i in one launch.
      grads_.begin();
      for (auto& b : bs_) grads_.add(b->grad().data(), b->value().cols(), static_cast<size_t>(k) * sizeof(Scalar));
      auto* table = static_cast<void* const*>(grads_.commit(dev(), ctx));
      GINN_HIP_CALL(ginn_hip_gemm_gathered(ctx, dtype_of<Scalar>(), internal::OP_T, internal::OP_N,
                                           static_cast<int>(k), static_cast<int>(total), static_cast<int>(m),
                                           a.data(), static_cast<int>(m), grad().data(), static_cast<int>(m),
                                           nullptr, 1.f, nullptr, 0, table, grads_.aligned()));
    } else if (with_grad > 0) {
      for (size_t i = 0; i < bs_.size(); ++i) {
        if (!bs_[i]->has_grad() || extents_[i] == 0) continue;
        GINN_HIP_CALL(ginn_hip_gemm(ctx, dtype_of<Scalar>(), internal::OP_T, internal::OP_N, static_cast<int>(k),
                                    static_cast<int>(extents_[i]), static_cast<int>(m), a.data(),
                                    static_cast<int>(m), grad().data() + offsets_[i] * m, static_cast<int>(m),
                                    1.f, bs_[i]->grad().data(), static_cast<int>(k)));
      }
    }
  }

  static std::vector<BaseNodePtr> all_ins(const NodePtr<Scalar>& a, const std::vector<NodePtr<Scalar>>& bs) {
    std::vector<BaseNodePtr> ins{a};
    ins.insert(ins.end(), bs.begin(), bs.end());
    return ins;
  }

 public:
  using BaseDataNode<Scalar>::dev;
  using BaseDataNode<Scalar>::value;
  using BaseDataNode<Scalar>::grad;

  GatherProdNode(const NodePtr<Scalar>& a, const std::vector<NodePtr<Scalar>>& bs)
      : BaseDataNode<Scalar>(all_ins(a, bs)), a_(a), bs_(bs) {
    GINN_ASSERT(!bs.empty(), "GatherProd needs at least one right operand");
  }

  const std::vector<Size>& offsets() const override { return offsets_; }
  const std::vector<Size>& extents() const override { return extents_; }
  // The left operand's gradient may be overwritten; the gathered ones are added
  // to by one launch for all of them, which has one beta.
  BaseNode::GradUse grad_use(size_t index) const override {
    return index == 0 ? BaseNode::GradUse::Overwrites : BaseNode::GradUse::Accumulates;
  }

  void set_ins(const std::vector<BaseNodePtr>& ins) override {
    GINN_ASSERT(ins.size() >= 2);
    BaseNode::ins_ = ins;
    a_ = dynamic_ptr_cast<Node<Scalar>>(ins[0]);
    bs_.clear();
    for (size_t i = 1; i < ins.size(); ++i) bs_.push_back(dynamic_ptr_cast<Node<Scalar>>(ins[i]));
  }
  std::string name() const override { return "GatherProd"; }
};

GINN_MAKE_SCALAR_FORWARDING_FACTORY(GatherProd);

// Per-slice product over all trailing dimensions (rank >= 3 inputs).
// On the HIP device the product is carried out when its value is first read: an operand that is a Permute
// whose copy is still pending is then read through its slices in ITS input's memory, and a Permute right
// behind this node has the result written permuted (node/slices.h); the gradients take the same ways back.
template <typename Scalar>
class BatchedProdNode : public BaseDataNode<Scalar>, public internal::SliceTaker<Scalar>, public PostponedValue {
  NodePtr<Scalar> a_, b_;
  mutable bool pending_ = false;  // forward() has run, the product has not
  bool grad_elsewhere_ = false;   // this pass's gradient lies in grad_view_ (take_grad_slices)
  internal::BatchView<Scalar> grad_view_;

  Tensor<Scalar>& raw_value() const { return const_cast<Tensor<Scalar>&>(BaseDataNode<Scalar>::value()); }
  // The slices of an operand's value: those a pending Permute offers, or the operand's own tensor.
  static internal::BatchView<Scalar> operand(const NodePtr<Scalar>& x) {
    internal::BatchView<Scalar> v;
    if (auto* p = dynamic_cast<internal::SliceProvider<Scalar>*>(x.get()); p && p->value_slices(v)) return v;
    return internal::contiguous_slices(x->value());
  }
  void multiply_into(const internal::BatchView<Scalar>& out) const {
    internal::batched_product(internal::ctx_of(raw_value()), out, operand(a_), false, operand(b_), false, false);
  }

  void forward_() override {
    const Shape sa = a_->shape(), sb = b_->shape();
    GINN_ASSERT(sa.size() >= 3 && sb.size() >= 3, "BatchedProd expects at least rank 3 inputs!");
    GINN_ASSERT(sa[1] == sb[0], "Mismatching inner dimensions in BatchedProd!");
    GINN_ASSERT(sa.size() == sb.size(), "Mismatching batch dimensions in BatchedProd!");
    for (size_t i = 2; i < sa.size(); ++i)
      GINN_ASSERT(sa[i] == sb[i], "Mismatching batch dimensions in BatchedProd!");
    Shape s = sb;
    s[0] = sa[0];
    raw_value().resize(s);
    grad_elsewhere_ = false;
    if (dev()->kind() == CPU) {
      pending_ = false;
      internal::cpu_batched_prod(raw_value(), a_->value(), b_->value());
      return;
    }
    internal::require_gpu(dev(), "BatchedProd");
    pending_ = raw_value().size() > 0;
  }
  void backward_() override {
    using namespace internal;
    if (dev()->kind() == CPU) {
      if (a_->has_grad())
        cpu_batched_prod(a_->grad(), grad(), b_->value(),
                         a_->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add, ProdTranspose::Second);
      if (b_->has_grad())
        cpu_batched_prod(b_->grad(), a_->value(), grad(),
                         b_->take_lazy_zero() ? ProdResult::Assign : ProdResult::Add, ProdTranspose::First);
      return;
    }
    const BatchView<Scalar> dy = grad_elsewhere_ ? grad_view_ : contiguous_slices(grad());
    grad_elsewhere_ = false;
    ginn_hip_ctx* ctx = ctx_of(raw_value());
    // Where the gradient of an operand goes: into the slices a Permute names inside its input's gradient
    // (this node being the only user of the Permute's), or into the operand's own gradient tensor.
    auto target = [](const NodePtr<Scalar>& x, bool& accumulate) {
      const bool fresh = x->take_lazy_zero();
      BatchView<Scalar> v;
      if (fresh)
        if (auto* p = dynamic_cast<SliceProvider<Scalar>*>(x.get()); p && p->grad_slices(v, accumulate)) return v;
      accumulate = !fresh;
      return contiguous_slices(x->grad());
    };
    if (a_->has_grad()) {  // dA = dY B^T
      bool acc = false;
      const BatchView<Scalar> da = target(a_, acc);
      batched_product(ctx, da, dy, false, operand(b_), true, acc);
    }
    if (b_->has_grad()) {  // dB = A^T dY
      bool acc = false;
      const BatchView<Scalar> db = target(b_, acc);
      batched_product(ctx, db, operand(a_), true, dy, false, acc);
    }
  }

 public:
  using BaseDataNode<Scalar>::grad;
  const Tensor<Scalar>& value() const override {
    if (pending_) {
      pending_ = false;
      multiply_into(internal::contiguous_slices(raw_value()));
    }
    return BaseDataNode<Scalar>::value();
  }
  using Node<Scalar>::value;
  void settle_value() override { (void)std::as_const(*this).value(); }
  Shape shape() const override { return BaseDataNode<Scalar>::value().shape(); }
  DevPtr dev() const override { return BaseDataNode<Scalar>::value().dev(); }

  bool product_pending() const override { return pending_; }
  void produce_into(const internal::BatchView<Scalar>& v) override {
    GINN_ASSERT(pending_, "BatchedProd: no product is pending");
    pending_ = false;
    multiply_into(v);
  }
  bool take_grad_slices(const internal::BatchView<Scalar>& v) override {
    if (dev()->kind() != GPU) return false;
    grad_view_ = v;
    grad_elsewhere_ = true;
    return true;
  }

  BatchedProdNode(const NodePtr<Scalar>& a, const NodePtr<Scalar>& b)
      : BaseDataNode<Scalar>({a, b}), a_(a), b_(b) {}
  BaseNode::GradUse grad_use(size_t) const override { return BaseNode::GradUse::Overwrites; }
  std::string name() const override { return "BatchedProd"; }
};

GINN_MAKE_SCALAR_FORWARDING_FACTORY(BatchedProd);

template <typename Left, typename Right>
auto operator*(const Ptr<Left>& a, const Ptr<Right>& b) {
  return Prod(a, b);
}

}  // namespace ginn

#endif  // GINN_NODE_PROD_H
