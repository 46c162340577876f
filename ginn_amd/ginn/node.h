// Graph core of the host layer: node handle, node base classes, Graph.
//
// Behaviour follows ginn/node.h:113-273: a node runs forward_() once until
// reset_forwarded(); backward() runs only when has_grad(); Graph orders the
// nodes reachable from a sink depth-first (inputs before users), seeds the
// sink gradient and walks the list in reverse.
#ifndef GINN_NODE_H
#define GINN_NODE_H

#include <memory>
#include <string>
#include <type_traits>
#include <algorithm>
#include <atomic>
#include <cstdint>
#include <utility>
#include <vector>

#include <ginn/tensor.h>

namespace ginn {

class BaseNode;

// Shared handle to a node; converts to handles of base classes.
template <typename NodeType>
class Ptr {
  static_assert(std::is_base_of_v<BaseNode, NodeType>, "Ptr only applies to classes deriving from BaseNode!");
  std::shared_ptr<NodeType> p_;

  template <typename T>
  friend class Ptr;

 public:
  using element_type = NodeType;

  Ptr() = default;
  Ptr(std::nullptr_t) {}
  Ptr(NodeType* raw) : p_(raw) {}
  Ptr(std::shared_ptr<NodeType> sp) : p_(std::move(sp)) {}
  template <typename Other, typename = std::enable_if_t<
                                std::is_convertible_v<std::shared_ptr<Other>, std::shared_ptr<NodeType>>>>
  Ptr(const Ptr<Other>& o) : p_(o.p_) {}
  template <typename Other>
  Ptr& operator=(const Ptr<Other>& o) {
    p_ = o.p_;
    return *this;
  }

  NodeType* operator->() const { return p_.get(); }
  NodeType& operator*() const { return *p_; }
  NodeType* get() const { return p_.get(); }
  const std::shared_ptr<NodeType>& as_shared_ptr() const { return p_; }
  bool operator==(const Ptr& o) const { return p_ == o.p_; }
  bool operator!=(const Ptr& o) const { return p_ != o.p_; }
  explicit operator bool() const { return static_cast<bool>(p_); }
};

template <typename NodeType, typename... Args>
auto make_ptr(Args&&... args) {
  return Ptr<NodeType>(std::make_shared<NodeType>(std::forward<Args>(args)...));
}

template <typename To, typename From>
auto dynamic_ptr_cast(const Ptr<From>& p) {
  return Ptr<To>(std::dynamic_pointer_cast<To>(p.as_shared_ptr()));
}

using BaseNodePtr = Ptr<BaseNode>;
using ConstBaseNodePtr = Ptr<const BaseNode>;

template <typename Container>
std::vector<BaseNodePtr> base_cast(Container&& v) {
  return std::vector<BaseNodePtr>(v.begin(), v.end());
}

template <typename Derived, typename Container>
std::vector<Ptr<Derived>> derived_cast(const Container& v);

// is_node_ptr_v<T>: T is some Ptr<...>.
template <typename T>
struct is_node_ptr : std::false_type {};
template <typename N>
struct is_node_ptr<Ptr<N>> : std::true_type {};
template <typename T>
inline constexpr bool is_node_ptr_v = is_node_ptr<std::decay_t<T>>::value;

// First element type of (possibly nested) containers of node handles.
template <typename T, typename = void>
struct innermost {
  using type = T;
};
template <typename T>
struct innermost<T, std::void_t<typename std::decay_t<T>::value_type>> {
  using type = typename innermost<typename std::decay_t<T>::value_type>::type;
};
template <typename T>
using innermost_t = typename innermost<T>::type;

// One elementwise operation on contiguous device memory, as a node describes
// it to the level executor (ginn/level_exec.h) instead of launching it: the
// executor merges the descriptions of all nodes of one height that agree in
// everything but the pointers into a single launch (ginn_hip_multi_apply).
struct LaunchDesc {
  int dtype = GINN_HIP_F32;
  int kind = GINN_HIP_MULTI_SUM;
  int act = GINN_HIP_ACT_IDENTITY;
  int accumulate = 0;
  float value = 0.f;
  int reserved = 0;  // keeps the struct free of padding: plans are compared bytewise
  size_t n = 0;
  void* dst = nullptr;
  const void* src[3] = {nullptr, nullptr, nullptr};
};
static_assert(sizeof(LaunchDesc) == 6 * 4 + 8 + 4 * 8, "LaunchDesc must not contain padding");

class BaseNode {
 protected:
  std::vector<BaseNodePtr> ins_;
  virtual void forward_() {}
  virtual void backward_() {}

 private:
  // Scratch of graph traversals (Graph, Autobatch, LevelExecutor).  A node
  // counts as visited by a traversal iff mark_epoch_ equals the traversal's
  // epoch, and mark_value_ is whatever the traversal keeps per node (a
  // height).  This replaces hash tables keyed by node address, which made up
  // a third of the host time of building and first running a graph of 100 k
  // nodes.  Like `forwarded`, the marks belong to the node: traversals of
  // graphs that share nodes must not run at the same time.
  mutable uint64_t mark_epoch_ = 0;
  mutable size_t mark_value_ = 0;
  // The pass (Graph / LevelExecutor id) in which this node is an input of
  // exactly one node, i.e. in which its gradient has a single writer; 0 = none.
  mutable uint64_t sole_user_pass_ = 0;

 public:
  bool forwarded = false;

  static uint64_t new_epoch() {
    static std::atomic<uint64_t> last{0};
    return ++last;
  }
  bool marked(uint64_t epoch) const { return mark_epoch_ == epoch; }
  void mark(uint64_t epoch, size_t value = 0) const {
    mark_epoch_ = epoch;
    mark_value_ = value;
  }
  size_t mark_value() const { return mark_value_; }
  uint64_t sole_user_pass() const { return sole_user_pass_; }
  void set_sole_user_pass(uint64_t pass) const { sole_user_pass_ = pass; }

  BaseNode() = default;
  BaseNode(std::vector<BaseNodePtr> ins) : ins_(std::move(ins)) {}
  template <typename DerivedPtr>
  BaseNode(std::vector<DerivedPtr> ins) : ins_(ins.begin(), ins.end()) {}
  virtual ~BaseNode() = default;

  const std::vector<BaseNodePtr>& ins() { return ins_; }
  std::vector<ConstBaseNodePtr> ins() const { return {ins_.begin(), ins_.end()}; }
  // The inputs of a const node without the copy the const ins() makes.
  const std::vector<BaseNodePtr>& inputs() const { return ins_; }
  const BaseNodePtr& in(size_t idx = 0) { return ins_.at(idx); }
  ConstBaseNodePtr in(size_t idx = 0) const { return ins_.at(idx); }

  // Rewiring hook used by Autobatch; nodes that support it override.
  virtual void set_ins(const std::vector<BaseNodePtr>&) {
    GINN_THROW("set_ins() for " + name() + " is not implemented!");
  }

  virtual DevPtr dev() const = 0;
  virtual Shape shape() const = 0;
  Shape shape2() const { return Tensor<>::reduce(shape(), 2); }
  Size rows() const { return shape2()[0]; }
  Size cols() const { return shape2()[1]; }
  Size size() const { return Tensor<>::size(shape()); }

  void forward() {
    if (forwarded) return;
    forward_();
    forwarded = true;
  }
  void backward() {
    if (has_grad()) backward_();
  }

  // Level-batched execution: a node whose work is elementwise on contiguous
  // memory may do its shape bookkeeping, append what it would have launched to
  // `out` and return true; false means "call forward() / backward() /
  // reset_grad() as usual".  describe_forward() is only called on nodes that
  // have not been forwarded, describe_backward() only when has_grad().
  virtual bool describe_forward(std::vector<LaunchDesc>&) { return false; }
  virtual bool describe_backward(std::vector<LaunchDesc>&) { return false; }
  virtual bool describe_reset_grad(std::vector<LaunchDesc>&) { return false; }

  virtual bool has_grad() const { return false; }
  virtual void init_grad() {}
  virtual void reset_grad() {}

  // ---- gradients that are cleared lazily -----------------------------------
  // A gradient with exactly one writer that can overwrite need not be zeroed
  // and then added to: Graph::reset_grad() (and the level executor's) only
  // flags such a gradient as "holds no value yet", and the writer, which asks
  // with take_lazy_zero() before it touches the gradient, then overwrites it
  // (a product runs with beta = 0).  Everything else sees zeros: reading a
  // flagged gradient through grad() clears it first.  The reference zeroes
  // every gradient in reset_grad() (ginn/node.h:218-222) and adds in every
  // backward; the values are the same, one write and one read of each such
  // gradient are not made.
  enum class GradUse {
    Accumulates,  // backward adds to the input's gradient (every node may)
    Overwrites,   // backward asks take_lazy_zero() of the input first and overwrites when told to
    Aliases       // this node's gradient IS the whole of the input's (views, in-place nodes)
  };
  // How backward() treats the gradient of input `index`.
  virtual GradUse grad_use(size_t /*index*/) const { return GradUse::Accumulates; }
  // The node holds gradient storage of its own that may be flagged.
  virtual bool owns_grad() const { return false; }
  // reset_grad() that may flag instead of zeroing.
  virtual void reset_grad_lazy() { reset_grad(); }
  // True exactly once after a lazy reset: the caller must now overwrite the
  // whole gradient.  Views and in-place nodes ask their input.
  virtual bool take_lazy_zero() { return false; }
  virtual bool lazy_zero() const { return false; }
  // Drops the flag without clearing: for an executor whose recorded launches
  // have overwritten the gradient.
  virtual void clear_lazy_zero() {}
  virtual void reset_forwarded() { forwarded = false; }
  virtual std::string name() const = 0;
};

template <typename Derived, typename Container>
std::vector<Ptr<Derived>> derived_cast(const Container& v) {
  std::vector<Ptr<Derived>> out;
  out.reserve(v.size());
  for (const auto& x : v) {
    auto d = dynamic_ptr_cast<Derived>(x);
    GINN_ASSERT(static_cast<bool>(d), "Failed to cast to a derived Node!");
    out.push_back(d);
  }
  return out;
}

template <typename ScalarType = Real>
class Node : public BaseNode {
 public:
  using Scalar = ScalarType;
  using BaseNode::BaseNode;

  virtual const Tensor<Scalar>& value() const = 0;
  virtual const Tensor<Scalar>& grad() const = 0;
  Tensor<Scalar>& value() { return const_cast<Tensor<Scalar>&>(std::as_const(*this).value()); }
  Tensor<Scalar>& grad() { return const_cast<Tensor<Scalar>&>(std::as_const(*this).grad()); }

  // The gradient tensor as it is, flagged or not: for views that map onto it.
  virtual Tensor<Scalar>& grad_storage() { return grad(); }

  DevPtr dev() const override { return value().dev(); }
  Shape shape() const override { return value().shape(); }

  void init_grad() override {
    GINN_ASSERT(forwarded, "Cannot init grad on non-forwarded nodes!");
    // shape(), not value(): a node that postpones the kernel behind its value is not asked for it here
    if (has_grad() && this->size() != grad().size()) grad().resize(this->shape());
  }
  void reset_grad() override {
    init_grad();
    if (has_grad()) grad().set_zero();
  }
  // Classes that override reset_grad() (views, aliases) also override this to
  // return false.
  bool describe_reset_grad(std::vector<LaunchDesc>& out) override {
    if constexpr (!is_floating_point_v<Scalar>) {
      return false;  // index tensors: no device arithmetic, no gradient
    } else {
      return describe_zero_grad(out);
    }
  }

 private:
  bool describe_zero_grad(std::vector<LaunchDesc>& out) {
    init_grad();
    if (!has_grad() || grad().size() == 0) return true;
    if (grad().dev()->kind() != GPU) {
      grad().set_zero();
      return true;
    }
    LaunchDesc d;
    d.dtype = dtype_of<Scalar>();
    d.kind = GINN_HIP_MULTI_FILL;
    d.n = static_cast<size_t>(grad().size());
    d.dst = grad().data();
    out.push_back(d);
    return true;
  }

 public:
  Scalar item() const { return value().item(); }
};

template <typename Scalar = Real>
using NodePtr = Ptr<Node<Scalar>>;
template <typename Scalar = Real>
using ConstNodePtr = Ptr<const Node<Scalar>>;

namespace internal {
inline bool& lazy_grad_reset_flag() {
  static bool on = true;
  return on;
}
// Zero fills made on demand because a flagged gradient was read or added to
// before anything overwrote it (process-wide, for tests and the executor).
inline std::atomic<size_t>& lazy_grad_settles() {
  static std::atomic<size_t> n{0};
  return n;
}
// Open while Graph::backward() / LevelExecutor::backward() runs on this thread.
// A row sum into the gradient of a leaf node (a bias, a LayerNorm scale) is two
// launches, partial sums and their fold; nothing reads such a gradient before
// the pass ends, so while a window is open the nodes postpone those folds
// (ginn_hip_defer_folds) and the pass runs them all as one launch at its end.
// Other work that only the end of the pass needs registers itself with
// at_close() (the gradient of a left operand shared by many merged products,
// node/prod.h).
class FoldWindow {
  static int& depth() {
    thread_local int d = 0;
    return d;
  }
  static std::vector<ginn_hip_ctx*>& touched() {
    thread_local std::vector<ginn_hip_ctx*> v;
    return v;
  }
  // fn(run): run != 0 does the postponed work, run == 0 only forgets it.
  static std::vector<void (*)(int)>& hooks() {
    thread_local std::vector<void (*)(int)> v;
    return v;
  }
  static uint64_t& pass_id() {
    thread_local uint64_t id = 0;
    return id;
  }

 public:
  // `pass`: the id of the Graph / LevelExecutor whose backward pass this is (0: unknown).
  explicit FoldWindow(uint64_t pass = 0) {
    if (++depth() == 1) pass_id() = pass;
  }
  FoldWindow(const FoldWindow&) = delete;
  FoldWindow& operator=(const FoldWindow&) = delete;
  ~FoldWindow() {
    if (--depth() != 0) return;
    pass_id() = 0;
    if (!hooks().empty()) {  // left by an exception: nothing stays queued
      for (auto* fn : hooks()) fn(0);
      hooks().clear();
    }
    if (!touched().empty()) {
      for (ginn_hip_ctx* c : touched()) (void)ginn_hip_flush_folds(c);
      touched().clear();
    }
  }
  static bool open() { return depth() > 0; }
  // The id of the outermost open pass on this thread; 0 when none or unknown.
  static uint64_t pass() { return depth() > 0 ? pass_id() : 0; }
  static void note(ginn_hip_ctx* ctx) {
    auto& v = touched();
    if (std::find(v.begin(), v.end(), ctx) == v.end()) v.push_back(ctx);
  }
  // first: ahead of the hooks registered so far (work that the others' work must find finished).
  static void at_close(void (*fn)(int), bool first = false) {
    auto& v = hooks();
    if (std::find(v.begin(), v.end(), fn) != v.end()) return;
    if (first) v.insert(v.begin(), fn);
    else v.push_back(fn);
  }
  // The end of the pass: the outermost window folds what was postponed.
  void close() {
    if (depth() != 1) return;
    std::vector<void (*)(int)> fns;
    fns.swap(hooks());
    for (size_t i = 0; i < fns.size(); ++i) {
      try {
        fns[i](1);
      } catch (...) {
        for (size_t j = i + 1; j < fns.size(); ++j) fns[j](0);
        throw;
      }
    }
    std::vector<ginn_hip_ctx*> v;
    v.swap(touched());
    for (ginn_hip_ctx* c : v) GINN_HIP_CALL(ginn_hip_flush_folds(c));
  }
};

// Products into the gradients of leaves (weights) beside the pass.  Every other product of a
// backward pass feeds the next node, one launch after the other, and many of them leave a
// quarter to a half of the CUs idle (144 or 192 tiles on 256 CUs); the gradient of a weight is
// needed by nobody until the pass ends.  While a pass runs, such a product is therefore enqueued
// on the GPU's second context: its stream waits for what the pass has enqueued so far (the
// product's operands), the pass goes on without waiting for it, and the end of the pass waits for
// the second stream.  The operands are a node's gradient and another node's value (or a buffer
// the node keeps), none of which changes before the next pass.  Same kernels, same results.
// The second stream is ordered behind what the pass had enqueued when the product was issued, not
// against what the pass enqueues later: a leaf qualifies only when the running pass has exactly ONE
// writer of its gradient (the leaf is an input of one node of the pass's graph, counted when the
// graph's gradients were last reset: BaseNode::sole_user_pass()).  A weight that several nodes
// share (tied weights, the cells of an unrolled recurrent net, a weight that is also summed by an
// Add) keeps all of its gradient writers on the pass's own stream.
inline bool& beside_pass_flag() {
  static bool on = true;
  return on;
}
// Launches sent to a second stream since the process began (for tests).
inline std::atomic<size_t>& beside_launches() {
  static std::atomic<size_t> n{0};
  return n;
}
class BesidePass {
  static std::vector<std::pair<ginn_hip_ctx*, ginn_hip_ctx*>>& joined() {
    thread_local std::vector<std::pair<ginn_hip_ctx*, ginn_hip_ctx*>> v;  // (main, beside) used in this pass
    return v;
  }
  static void join(int) {  // also when the pass ends by an exception
    std::vector<std::pair<ginn_hip_ctx*, ginn_hip_ctx*>> v;
    v.swap(joined());
    for (auto& [main, beside] : v) {
      int ordered = 0;
      (void)ginn_hip_ctx_wait_for(main, beside, &ordered);
      if (!ordered) (void)ginn_hip_sync(beside);  // cannot happen: no capture began since the product
    }
  }

 public:
  static constexpr double kWorthIt = 1e9;  // flops below which the two events cost more than the overlap gains
  // The context to enqueue a product of `flops` into the gradient of `target` on.
  static ginn_hip_ctx* ctx_for(const BaseNode& target, const DevPtr& dev, double flops) {
    const size_t idx = dev->id().idx;
    ginn_hip_ctx* main = contexts().at(idx);
    if (!beside_pass_flag() || !FoldWindow::open() || !target.inputs().empty() || flops < kWorthIt) return main;
    if (FoldWindow::pass() == 0 || target.sole_user_pass() != FoldWindow::pass()) return main;
    ginn_hip_ctx* beside = contexts().beside(idx);
    int ordered = 0;
    GINN_HIP_CALL(ginn_hip_ctx_wait_for(beside, main, &ordered));
    if (!ordered) return main;  // a device graph is being recorded: one stream
    auto& v = joined();
    if (std::find(v.begin(), v.end(), std::make_pair(main, beside)) == v.end()) v.emplace_back(main, beside);
    FoldWindow::at_close(&join, /*first=*/true);
    ++beside_launches();
    return beside;
  }
};

// Around one library call whose row sums go into the gradient of `target`.
class PostponeFolds {
  ginn_hip_ctx* ctx_ = nullptr;

 public:
  template <typename... Targets>
  PostponeFolds(ginn_hip_ctx* ctx, const Targets&... targets) {
    const bool leaves = (... && targets.inputs().empty());
    if (FoldWindow::open() && leaves && ginn_hip_defer_folds(ctx, 1) == 0) {
      ctx_ = ctx;
      FoldWindow::note(ctx);
    }
  }
  PostponeFolds(const PostponeFolds&) = delete;
  PostponeFolds& operator=(const PostponeFolds&) = delete;
  ~PostponeFolds() {
    if (ctx_) (void)ginn_hip_defer_folds(ctx_, 0);
  }
};

// While set, every gradient whose flag is taken is noted here (the level
// executor tells apart the flags that recorded launches consume).
inline std::vector<BaseNode*>*& lazy_take_log() {
  thread_local std::vector<BaseNode*>* log = nullptr;
  return log;
}
}  // namespace internal

// Whether products into the gradients of weights may run on the GPU's second stream while a
// backward pass runs (internal::BesidePass); on by default.
inline void set_beside_pass(bool on) { internal::beside_pass_flag() = on; }
inline bool beside_pass() { return internal::beside_pass_flag(); }

// Whether reset_grad() of Graph and LevelExecutor may flag gradients instead of
// zeroing them (BaseNode::GradUse); on by default.
inline void set_lazy_grad_reset(bool on) { internal::lazy_grad_reset_flag() = on; }
inline bool lazy_grad_reset() { return internal::lazy_grad_reset_flag(); }

// For a node list in graph order (inputs first): out[i] != 0 iff the gradient
// of list[i] may be flagged instead of zeroed.  That takes storage of its own,
// exactly one use as an input within the list, and a user that overwrites --
// directly, or through a chain of views and in-place nodes each with one use.
// With a pass id, every leaf of the list that is an input of exactly one node
// is also noted as having a single gradient writer in that pass
// (internal::BesidePass), and every other leaf as having several.
inline std::vector<unsigned char> lazy_grad_candidates(const std::vector<BaseNodePtr>& list, uint64_t pass = 0) {
  const size_t n = list.size();
  std::vector<unsigned char> out(n, 0);
  if (!internal::lazy_grad_reset_flag() && pass == 0) return out;
  const uint64_t epoch = BaseNode::new_epoch();
  for (size_t i = 0; i < n; ++i) list[i]->mark(epoch, i);
  std::vector<uint32_t> uses(n, 0), user(n, 0), slot(n, 0);
  for (size_t u = 0; u < n; ++u) {
    const auto& ins = list[u]->inputs();
    for (size_t k = 0; k < ins.size(); ++k) {
      if (!ins[k]->marked(epoch)) continue;
      const size_t j = ins[k]->mark_value();
      ++uses[j];
      user[j] = static_cast<uint32_t>(u);
      slot[j] = static_cast<uint32_t>(k);
    }
  }
  if (pass != 0)
    for (size_t j = 0; j < n; ++j)
      if (list[j]->inputs().empty()) list[j]->set_sole_user_pass(uses[j] == 1 ? pass : 0);
  if (!internal::lazy_grad_reset_flag()) return out;
  std::vector<unsigned char> overwritten(n, 0);  // by the one user, were the gradient flagged
  for (size_t j = n; j-- > 0;) {                 // users come later in the list
    BaseNode& node = *list[j];
    if (uses[j] != 1 || !node.has_grad()) continue;
    BaseNode& u = *list[user[j]];
    if (!u.has_grad()) continue;
    const BaseNode::GradUse use = u.grad_use(slot[j]);
    if (use == BaseNode::GradUse::Overwrites) overwritten[j] = 1;
    else if (use == BaseNode::GradUse::Aliases) overwritten[j] = overwritten[user[j]];
    out[j] = overwritten[j] && node.owns_grad();
  }
  return out;
}

// An in-place step (scale, mask) that postpones its work until somebody reads
// its value: a Softmax directly after it then does scale, mask and softmax as
// one launch over the scores (ginn_hip_scaled_masked_softmax_fwd) instead of
// three.  Whoever else reads the value first triggers the step as usual.
class PendingInPlace {
 public:
  enum class Step { Scale, Mask };
  virtual ~PendingInPlace() = default;
  virtual Step pending_step() const = 0;
  virtual bool pending() const = 0;
  virtual void take_pending() = 0;             // the caller does the step itself
  virtual float pending_value() const = 0;     // the factor, or the value for masked entries
  virtual BaseNode* pending_mask() const { return nullptr; }
  virtual BaseNode* pending_input() const = 0;  // the node whose storage the step writes over
  virtual void skip_next_backward() = 0;        // the caller has done this step's backward too
  // Runs the step now if it is still pending.  Graph::forward() and
  // LevelExecutor::forward() call this for every such node when the pass ends,
  // so that the storage written over holds the final contents for any reader
  // once forward() has returned (ginn/node/inplace.h:104-123, 152-212).
  virtual void settle() = 0;
};

// A node that postpones the kernel behind its value until value() is called (LayerNorm, Permute,
// BatchedProd), so that the node reading it can do both steps in one.  Every reader that runs as code of
// its own calls value() and gets it.  A frozen LevelExecutor replays the work of all other readers from
// what it recorded, calling nothing: it therefore asks such a node for its value right after forward()
// when one of the node's readers is among the replayed ones (settle_value()).
class PostponedValue {
 public:
  virtual ~PostponedValue() = default;
  virtual void settle_value() = 0;
};

class Graph {
  std::vector<BaseNodePtr> list_;
  std::vector<PendingInPlace*> pending_steps_;  // the nodes of list_ that may postpone their work
  uint64_t id_ = BaseNode::new_epoch();  // names this graph's passes (copies hold the same list)

  // Depth-first, a node after all of its inputs, without recursion: the
  // depth of a graph is its longest path (a recurrent net unrolled over
  // thousands of steps), not something the call stack should carry.
  void visit(const BaseNodePtr& sink, uint64_t epoch) {
    std::vector<std::pair<BaseNodePtr, size_t>> stack;  // node, next input to look at
    sink->mark(epoch);
    stack.emplace_back(sink, 0);
    while (!stack.empty()) {
      const BaseNodePtr node = stack.back().first;
      const auto& ins = node->ins();
      if (stack.back().second < ins.size()) {
        const BaseNodePtr& in = ins[stack.back().second++];
        if (!in->marked(epoch)) {
          in->mark(epoch);
          stack.emplace_back(in, 0);
        }
      } else {
        list_.push_back(node);
        stack.pop_back();
      }
    }
  }

 public:
  Graph(BaseNodePtr sink) {
    // A node is appended after all of its inputs; it is marked on entry,
    // which is equivalent for an acyclic graph.
    visit(sink, BaseNode::new_epoch());
    for (auto& e : list_)
      if (auto* p = dynamic_cast<PendingInPlace*>(e.get())) pending_steps_.push_back(p);
  }

  // In-place steps that nobody has asked for by the end of the pass run then
  // (PendingInPlace): after forward() every tensor holds its final contents.
  Graph& forward() {
    for (auto& e : list_) e->forward();
    for (PendingInPlace* p : pending_steps_) p->settle();
    return *this;
  }

  // Seeds the sink gradient with loss_coeff (whatever its shape) and
  // back-propagates; reset_grad() must have been called (ginn/node.h:237-254).
  Graph& backward(double loss_coeff = 1) {
    GINN_ASSERT(!list_.empty());
    if (auto s = dynamic_ptr_cast<Node<Real>>(list_.back())) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(static_cast<Real>(loss_coeff));
    } else if (auto s = dynamic_ptr_cast<Node<Half>>(list_.back())) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(Half(static_cast<float>(loss_coeff)));
    } else if (auto s = dynamic_ptr_cast<Node<BFloat16>>(list_.back())) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(BFloat16(static_cast<float>(loss_coeff)));
    } else {
      GINN_THROW("Unexpected scalar type in sink node!");
    }
    internal::FoldWindow folds(id_);
    for (auto it = list_.rbegin(); it != list_.rend(); ++it)
      if ((*it)->has_grad()) (*it)->backward();
    folds.close();
    return *this;
  }

  Graph& init_grad() {
    for (auto& e : list_) e->init_grad();
    return *this;
  }
  // Gradients with a single overwriting user are flagged, not zeroed
  // (BaseNode::GradUse); all others are zeroed as in ginn/node.h:218-222.
  Graph& reset_grad() {
    const std::vector<unsigned char> lazy = lazy_grad_candidates(list_, id_);
    for (size_t i = 0; i < list_.size(); ++i) {
      if (lazy[i]) list_[i]->reset_grad_lazy();
      else list_[i]->reset_grad();
    }
    return *this;
  }
  Graph& reset_forwarded() {
    for (auto& e : list_) e->reset_forwarded();
    return *this;
  }

  const std::vector<BaseNodePtr>& nodes() const { return list_; }
  BaseNodePtr sink() const { return list_.back(); }
};

// Factory generators (ginn/node.h:279-326): X(...) makes an XNode; FixedX(...)
// additionally switches its gradient off.
#define GINN_MAKE_FACTORY(f)                                                   \
  template <typename... Args>                                                  \
  auto f(Args&&... args) {                                                     \
    return ::ginn::make_ptr<f##Node>(std::forward<Args>(args)...);             \
  }                                                                            \
  template <typename... Args>                                                  \
  auto Fixed##f(Args&&... args) {                                              \
    auto n = ::ginn::make_ptr<f##Node>(std::forward<Args>(args)...);           \
    n->set_has_grad(false);                                                    \
    return n;                                                                  \
  }                                                                            \
  static_assert(true, "semicolon")

#define GINN_MAKE_TEMPLATE_FACTORY(f)                                          \
  template <typename Scalar = ::ginn::Real, typename... Args>                  \
  auto f(Args&&... args) {                                                     \
    return ::ginn::make_ptr<f##Node<Scalar>>(std::forward<Args>(args)...);     \
  }                                                                            \
  template <typename Scalar = ::ginn::Real, typename... Args>                  \
  auto Fixed##f(Args&&... args) {                                              \
    auto n = ::ginn::make_ptr<f##Node<Scalar>>(std::forward<Args>(args)...);   \
    n->set_has_grad(false);                                                    \
    return n;                                                                  \
  }                                                                            \
  static_assert(true, "semicolon")

// f(first, rest...) builds fNode<Scalar> with the Scalar of the first argument
// (a node handle or a container of node handles).
#define GINN_MAKE_SCALAR_FORWARDING_FACTORY(f)                                 \
  template <typename Arg, typename... Args>                                    \
  auto f(Arg&& arg, Args&&... args) {                                          \
    using Handle = ::ginn::innermost_t<Arg>;                                   \
    using Scalar = typename std::decay_t<Handle>::element_type::Scalar;        \
    return ::ginn::make_ptr<f##Node<Scalar>>(std::forward<Arg>(arg), std::forward<Args>(args)...); \
  }                                                                            \
  static_assert(true, "semicolon")

}  // namespace ginn

#endif  // GINN_NODE_H
