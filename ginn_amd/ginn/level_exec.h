// Level-batched execution of a graph on the HIP device.
//
// Graph::forward() runs one node after the other, and a node is one or more
// kernel launches.  Dynamic graphs (a recurrent cell unrolled over hundreds of
// sequences, a tree) consist of thousands of small nodes, so the launches --
// not the arithmetic -- set the pace.  Autobatch (ginn/autobatch.h:42-202)
// removes that for the products; LevelExecutor does it for the element-wise
// nodes around them without rewriting the graph: nodes are ordered by height
// (inputs strictly below their users, so the nodes of one height are
// independent), every node of a height that can describe its work as an
// element-wise operation does so (BaseNode::describe_*), the descriptions of
// a height become ONE launch over a table of operation records
// (ginn_hip_multi_mixed), and everything else runs as usual.  Values,
// gradients and node objects are exactly those of plain execution.
//
// The grouping of a level and its pointer tables (device memory owned by the
// executor) are kept as a plan and replayed as long as the nodes of the level
// describe the same operations on the same memory, i.e. on every pass over a
// static graph after the first.
#ifndef GINN_LEVEL_EXEC_H
#define GINN_LEVEL_EXEC_H

#include <algorithm>
#include <cstddef>
#include <cstring>
#include <functional>
#include <utility>
#include <unordered_set>

#include <ginn/node.h>

namespace ginn {

class LevelExecutor {
  // A description is uploaded as the operation record of the C ABI.
  static_assert(sizeof(LaunchDesc) == sizeof(ginn_hip_multi_op) &&
                    offsetof(LaunchDesc, n) == offsetof(ginn_hip_multi_op, n) &&
                    offsetof(LaunchDesc, dst) == offsetof(ginn_hip_multi_op, dst) &&
                    offsetof(LaunchDesc, src) == offsetof(ginn_hip_multi_op, src) &&
                    offsetof(LaunchDesc, value) == offsetof(ginn_hip_multi_op, value),
                "LaunchDesc and ginn_hip_multi_op must have one layout");
  struct Key {  // what a reduction launch needs beside its table
    int dtype = GINN_HIP_F32;
    size_t n = 0;
  };
  struct Launch {
    Key key;
    size_t count;   // operations
    size_t offset;  // of its table, in pointers from the start of the blob
    void* reduce_dst = nullptr;  // set: one reduction of `count` sources (table at offset) into this
    size_t zero_max = 0;         // set: zero fill of `count` regions (pointers at offset, byte counts at aux)
    size_t aux = 0;
    size_t mixed_max = 0;        // set: `count` operation records at offset, the longest of this many elements
    bool late = false;           // a reduction that runs as part of one at the end of the pass (LateReduce)
  };
  // What one flush (the described nodes of one level and pass) turned into.
  // As long as the nodes describe the same operations on the same memory --
  // every pass over a static graph after the first -- the plan is replayed
  // without regrouping or uploading anything.
  struct Plan {
    std::vector<LaunchDesc> descs;
    std::vector<Launch> launches;
    std::vector<const void*> blob;  // host copy of the tables
    void* dev = nullptr;  // all tables of the plan, one allocation
    size_t capacity = 0;  // bytes
  };
  // Several consecutive steps of a frozen pass as one launch: the operation
  // records of their launches regrouped into independent chains (fuse()).
  struct Chain {
    void* dev = nullptr;  // chain ranges, then operation records
    size_t chains = 0, ops = 0, stages = 0;
  };
  // A frozen, fused pass: nodes that run themselves, plans and chains in order.
  struct Item {
    std::vector<BaseNode*> direct;
    long plan = -1;  // with [first, first + count) of its launches
    size_t first = 0, count = 0;
    long chain = -1;
  };
  // One launch of a plan of the pass being fused.
  struct LaunchRef {
    long plan;
    size_t index;
  };
  // The reductions of a frozen backward pass into the gradient of one leaf (a
  // bias that every step of every sequence adds to: one reduction per level)
  // as ONE reduction over all their sources at the end of the pass.  Nothing
  // reads a leaf's gradient during the pass, and a source that is gradient
  // storage owned by its node is not written again once that node has run
  // (only nodes above it can alias it), so the sum is the same.
  struct LateReduce {
    void* dst = nullptr;
    int dtype = GINN_HIP_F32;
    size_t n = 0;
    std::vector<const void*> srcs;
    std::vector<Launch*> members;
    void* dev = nullptr;
  };
  std::vector<LateReduce> late_reduces_;
  std::vector<Chain> chains_;
  std::vector<Item> fused_[3];
  bool fused_ready_ = false;

  std::vector<BaseNodePtr> list_;               // graph order (inputs first)
  uint64_t id_ = BaseNode::new_epoch();         // names this executor's passes (internal::BesidePass)
  std::vector<PendingInPlace*> pending_steps_;  // nodes that may postpone their work past their forward()
  std::vector<std::vector<BaseNode*>> levels_;  // by height, ascending
  DevPtr dev_;
  ginn_hip_ctx* ctx_ = nullptr;
  std::vector<Plan> plans_[3];  // per pass, in flush order
  size_t cursor_ = 0;
  // One step = one level of a pass (the whole of reset_grad is one step): the
  // nodes that ran themselves, in order, then the plan of the described ones.
  struct Step {
    std::vector<BaseNode*> direct;
    long plan = -1;  // index into plans_[pass]; -1: nothing was described
  };
  std::vector<Step> steps_[3];
  std::vector<LaunchDesc> descs_;  // scratch of the pass under way (keeps its capacity)
  // Nodes whose gradient reset_grad() flags instead of zeroing (BaseNode::GradUse),
  // as of the last pass that was not frozen.
  std::vector<BaseNode*> lazy_;
  // Those of them whose flag a node takes while it runs itself: only these
  // are flagged again in frozen passes (a recorded launch asks nothing).
  std::vector<BaseNode*> lazy_direct_;
  std::vector<BaseNode*> taken_by_plans_;
  // A flagged gradient was zeroed on demand while a node described its work:
  // that fill is in no plan, so the passes cannot be replayed from plans.
  bool unplanned_fill_ = false;
  bool frozen_ = false;
  // Nodes that postpone the kernel behind their value (PostponedValue) and have a reader whose work a
  // frozen pass replays from the recording: asked for their value right after forward() (freeze()).
  std::unordered_set<BaseNode*> settle_after_forward_;
  ginn_hip_graph* pass_graph_ = nullptr;  // a recorded frozen pass (record_pass())

  void drop_graph() {
    if (pass_graph_) ginn_hip_graph_destroy(pass_graph_);
    pass_graph_ = nullptr;
  }
  size_t launches_ = 0, described_ = 0, rebuilt_ = 0;

  enum Pass { kForward = 0, kReset = 1, kBackward = 2 };
  static constexpr size_t kReduceFrom = 4;  // users of one destination that make a reduction worthwhile

  void build_levels() {
    const uint64_t epoch = BaseNode::new_epoch();  // marks carry heights
    size_t tallest = 0;
    for (auto& n : list_) {  // list_ is topologically sorted
      size_t h = 0;
      for (auto& in : n->ins()) {
        GINN_ASSERT(in->marked(epoch), "LevelExecutor: the graph's node list is not in topological order");
        h = std::max(h, in->mark_value());
      }
      n->mark(epoch, h + 1);
      tallest = std::max(tallest, h + 1);
    }
    std::vector<size_t> population(tallest, 0);
    for (auto& n : list_) ++population[n->mark_value() - 1];
    levels_.assign(tallest, {});
    for (size_t h = 0; h < tallest; ++h) levels_[h].reserve(population[h]);
    for (auto& n : list_) levels_[n->mark_value() - 1].push_back(n.get());
  }

  static Key key_of(const LaunchDesc& d) { return Key{d.dtype, d.n}; }

  // Turns the descriptions of one step into launches: one zero fill for all
  // cleared regions, one reduction per destination with many users, and one
  // launch for all other operations (more when destinations overlap).
  // Uploads the tables.
  void rebuild(Plan& plan, const std::vector<LaunchDesc>& descs) {
    ++rebuilt_;
    plan.descs = descs;
    plan.launches.clear();
    std::vector<const void*>& blob = plan.blob;
    blob.clear();
    // Three kinds of descriptions: zero fills (the gradients reset_grad()
    // clears), candidates for a reduction (one source added into a
    // destination), and all others.
    std::vector<const LaunchDesc*> zeros, adds, members;
    for (const auto& d : plan.descs) {
      if (d.n == 0) continue;
      if (d.kind == GINN_HIP_MULTI_FILL && !d.accumulate && d.value == 0.f) zeros.push_back(&d);
      else if (d.kind == GINN_HIP_MULTI_SUM && d.accumulate && d.src[0] && !d.src[1] && !d.src[2]) adds.push_back(&d);
      else members.push_back(&d);
    }
    // All zero fills, whatever their sizes and types: one launch over a table
    // of regions (at most 65535 regions per launch).
    if (zeros.size() >= 2) {
      const size_t count = zeros.size(), at = blob.size();
      blob.resize(at + 2 * count, nullptr);
      size_t largest = 0;
      for (size_t i = 0; i < count; ++i) {
        const size_t bytes = zeros[i]->n * (zeros[i]->dtype == GINN_HIP_F32 ? 4 : 2);
        blob[at + i] = zeros[i]->dst;
        blob[at + count + i] = reinterpret_cast<const void*>(static_cast<uintptr_t>(bytes));
        largest = std::max(largest, bytes);
      }
      for (size_t done = 0; done < count; done += 65535) {
        Launch l{Key{}, std::min<size_t>(65535, count - done), at + done};
        l.zero_max = largest;
        l.aux = at + count + done;
        plan.launches.push_back(l);
      }
    } else {
      members.insert(members.end(), zeros.begin(), zeros.end());
    }
    // Many users adding into the gradient of one node (a bias shared by all
    // steps of all sequences): one reduction instead of one launch each.
    // Everything else of the level, whatever it computes, shares launches.
    std::stable_sort(adds.begin(), adds.end(), [](const LaunchDesc* a, const LaunchDesc* b) {
      if (a->dst != b->dst) return std::less<const void*>()(a->dst, b->dst);
      if (a->n != b->n) return a->n < b->n;
      return a->dtype < b->dtype;
    });
    for (size_t i = 0; i < adds.size();) {
      size_t j = i;
      while (j < adds.size() && adds[j]->dst == adds[i]->dst && adds[j]->n == adds[i]->n &&
             adds[j]->dtype == adds[i]->dtype)
        ++j;
      if (j - i >= kReduceFrom) {
        const size_t at = blob.size();
        for (size_t u = i; u < j; ++u) blob.push_back(adds[u]->src[0]);
        Launch l{key_of(*adds[i]), j - i, at};
        l.reduce_dst = adds[i]->dst;
        plan.launches.push_back(l);
      } else {
        members.insert(members.end(), adds.begin() + i, adds.begin() + j);
      }
      i = j;
    }
    // Operations whose destinations overlap (two users adding into the
    // gradient of one node) go into successive launches: with destinations
    // ascending, a member fits a round iff it begins at or after the end of
    // everything already in that round.
    std::stable_sort(members.begin(), members.end(), [](const LaunchDesc* a, const LaunchDesc* b) {
      return std::less<const void*>()(a->dst, b->dst);
    });
    std::vector<std::vector<const LaunchDesc*>> rounds;
    std::vector<uintptr_t> round_end;
    for (const LaunchDesc* d : members) {
      const uintptr_t begin = reinterpret_cast<uintptr_t>(d->dst);
      const uintptr_t end = begin + d->n * (d->dtype == GINN_HIP_F32 ? 4 : 2);
      size_t r = 0;
      while (r < rounds.size() && (round_end[r] > begin || rounds[r].size() >= 65535)) ++r;
      if (r == rounds.size()) {
        rounds.emplace_back();
        round_end.push_back(0);
      }
      rounds[r].push_back(d);
      round_end[r] = std::max(round_end[r], end);
    }
    for (auto& round : rounds) {
      const size_t count = round.size(), at = blob.size();
      blob.resize(at + kSlots * count, nullptr);
      Launch l{Key{}, count, at};
      for (size_t i = 0; i < count; ++i) {
        std::memcpy(&blob[at + kSlots * i], round[i], sizeof(LaunchDesc));
        l.mixed_max = std::max(l.mixed_max, round[i]->n);
      }
      plan.launches.push_back(l);
    }
    const size_t bytes = blob.size() * sizeof(void*);
    if (bytes == 0) return;
    if (plan.capacity < bytes) {
      if (plan.dev) dev_->free(plan.dev);
      plan.dev = dev_->alloc(bytes);
      plan.capacity = bytes;
    }
    GINN_HIP_CALL(ginn_hip_memcpy_h2d(ctx_, plan.dev, blob.data(), bytes));
    // The blob is reused by the next rebuild and the copy is only ordered on the
    // stream: wait for it (plans are rebuilt when a graph changes, not per pass).
    GINN_HIP_CALL(ginn_hip_sync(ctx_));
  }

  void launch(const Plan& plan) { launch(plan, 0, plan.launches.size()); }

  void launch(const Plan& plan, size_t first, size_t count) {
    size_t skipped = 0;
    for (size_t li = first; li < first + count; ++li) {
      const Launch& l = plan.launches[li];
      if (l.zero_max) {
        const void* const* tables = static_cast<const void* const*>(plan.dev);
        GINN_HIP_CALL(ginn_hip_multi_zero(ctx_, static_cast<int>(l.count), const_cast<void* const*>(tables + l.offset),
                                          reinterpret_cast<const size_t*>(tables + l.aux), l.zero_max));
        continue;
      }
      if (l.reduce_dst) {
        if (l.late) {
          ++skipped;
          continue;
        }
        GINN_HIP_CALL(ginn_hip_multi_reduce(ctx_, static_cast<ginn_hip_dtype>(l.key.dtype), l.key.n,
                                            static_cast<int>(l.count),
                                            static_cast<const void* const*>(plan.dev) + l.offset, l.reduce_dst, 1));
        continue;
      }
      GINN_HIP_CALL(ginn_hip_multi_mixed(
          ctx_, static_cast<int>(l.count),
          reinterpret_cast<const ginn_hip_multi_op*>(static_cast<const void* const*>(plan.dev) + l.offset),
          l.mixed_max));
    }
    launches_ += count - skipped;
  }

  // Gradient storage [begin, end) of a node, whatever its scalar.
  static bool grad_range(BaseNode& n, uintptr_t& begin, uintptr_t& end) {
    auto of = [&](auto* t) {
      if (!t) return false;
      auto& g = t->grad_storage();
      begin = reinterpret_cast<uintptr_t>(g.data());
      end = begin + static_cast<size_t>(g.size()) * sizeof(*g.data());
      return true;
    };
    return of(dynamic_cast<Node<Real>*>(&n)) || of(dynamic_cast<Node<Half>*>(&n)) ||
           of(dynamic_cast<Node<BFloat16>*>(&n));
  }

  void drop_late_reductions() {
    for (LateReduce& r : late_reduces_) {
      for (Launch* l : r.members) l->late = false;
      if (r.dev) {
        try {
          dev_->free(r.dev);
        } catch (...) {
        }
      }
    }
    late_reduces_.clear();
  }

  // freeze(): see LateReduce.
  void plan_late_reductions() {
    drop_late_reductions();
    std::vector<std::pair<uintptr_t, uintptr_t>> owned;  // gradient storage that belongs to its node
    std::vector<uintptr_t> leaves;                        // ... of nodes without inputs
    for (auto& n : list_) {
      if (!n->has_grad() || !n->owns_grad()) continue;
      uintptr_t b = 0, e = 0;
      if (!grad_range(*n, b, e) || b == e) continue;
      owned.emplace_back(b, e);
      if (n->ins().empty()) leaves.push_back(b);
    }
    std::sort(owned.begin(), owned.end());
    std::sort(leaves.begin(), leaves.end());
    auto is_owned = [&](const void* p, size_t bytes) {
      const uintptr_t at = reinterpret_cast<uintptr_t>(p);
      auto it = std::upper_bound(owned.begin(), owned.end(), std::make_pair(at, ~uintptr_t(0)));
      if (it == owned.begin()) return false;
      --it;
      return at >= it->first && at + bytes <= it->second;
    };
    for (const Step& step : steps_[kBackward]) {
      if (step.plan < 0) continue;
      Plan& plan = plans_[kBackward][static_cast<size_t>(step.plan)];
      for (Launch& l : plan.launches) {
        if (!l.reduce_dst) continue;
        if (!std::binary_search(leaves.begin(), leaves.end(), reinterpret_cast<uintptr_t>(l.reduce_dst))) continue;
        const size_t bytes = l.key.n * (l.key.dtype == GINN_HIP_F32 ? 4 : 2);
        bool ok = true;
        for (size_t i = 0; i < l.count && ok; ++i) ok = is_owned(plan.blob[l.offset + i], bytes);
        if (!ok) continue;
        LateReduce* into = nullptr;
        for (LateReduce& r : late_reduces_)
          if (r.dst == l.reduce_dst && r.dtype == l.key.dtype && r.n == l.key.n) into = &r;
        if (!into) {
          late_reduces_.emplace_back();
          into = &late_reduces_.back();
          into->dst = l.reduce_dst;
          into->dtype = l.key.dtype;
          into->n = l.key.n;
        }
        into->srcs.insert(into->srcs.end(), plan.blob.begin() + static_cast<long>(l.offset),
                          plan.blob.begin() + static_cast<long>(l.offset + l.count));
        into->members.push_back(&l);
      }
    }
    // One reduction alone gains nothing by waiting.
    late_reduces_.erase(std::remove_if(late_reduces_.begin(), late_reduces_.end(),
                                       [](const LateReduce& r) {
                                         return r.members.size() < 2 || r.srcs.size() > 0x7fffffffu;
                                       }),
                        late_reduces_.end());
    for (LateReduce& r : late_reduces_) {
      r.dev = dev_->alloc(r.srcs.size() * sizeof(void*));
      GINN_HIP_CALL(ginn_hip_memcpy_h2d(ctx_, r.dev, r.srcs.data(), r.srcs.size() * sizeof(void*)));
      for (Launch* l : r.members) l->late = true;
    }
    if (!late_reduces_.empty()) GINN_HIP_CALL(ginn_hip_sync(ctx_));  // pageable copies: the tables have arrived
  }

  void run_late_reductions() {
    for (const LateReduce& r : late_reduces_) {
      GINN_HIP_CALL(ginn_hip_multi_reduce(ctx_, static_cast<ginn_hip_dtype>(r.dtype), r.n,
                                          static_cast<int>(r.srcs.size()),
                                          static_cast<const void* const*>(r.dev), r.dst, 1));
      ++launches_;
    }
  }

  // Ends a step: launches what its nodes described (reusing the plan of the
  // previous pass when they described the same) and notes the plan in `step`.
  void flush(Pass pass, Step& step) {
    step.plan = -1;
    if (descs_.empty()) return;
    described_ += descs_.size();
    auto& plans = plans_[pass];
    if (cursor_ == plans.size()) plans.emplace_back();
    step.plan = static_cast<long>(cursor_);
    Plan& plan = plans[cursor_++];
    const bool same = plan.descs.size() == descs_.size() &&
                      std::memcmp(plan.descs.data(), descs_.data(), descs_.size() * sizeof(LaunchDesc)) == 0;
    if (!same) rebuild(plan, descs_);
    launch(plan);
    descs_.clear();
  }

  Step& begin_step(Pass pass, size_t index) {
    auto& steps = steps_[pass];
    if (steps.size() <= index) steps.resize(index + 1);
    steps[index].direct.clear();
    return steps[index];
  }

  static constexpr size_t kSlots = sizeof(ginn_hip_multi_op) / sizeof(void*);
  static constexpr size_t kChainWork = 65536;  // elements a chain may touch in all of its operations

  void drop_chains() {
    for (Chain& c : chains_)
      if (c.dev) {
        try {
          dev_->free(c.dev);
        } catch (...) {
        }
      }
    chains_.clear();
    for (auto& f : fused_) f.clear();
    fused_ready_ = false;
  }

  // Tries to turn the launches of the plans `run` (in order) into one chain
  // launch.  Operations are joined into a chain when one writes memory that
  // the other reads or writes; the launch they came from is their stage.
  // Gives up (returns -1) when a chain would be long: then the operations are
  // large and a launch per stage costs nothing by comparison.
  // The operation records of the mixed launches `run`, stage = position in run.
  std::vector<LaunchDesc> records_of(Pass pass, const std::vector<LaunchRef>& run) const {
    std::vector<LaunchDesc> ops;
    int stage = 0;
    for (const LaunchRef& ref : run) {
      const Plan& plan = plans_[pass][static_cast<size_t>(ref.plan)];
      const Launch& l = plan.launches[ref.index];
      for (size_t i = 0; i < l.count; ++i) {
        LaunchDesc d;
        std::memcpy(static_cast<void*>(&d), &plan.blob[l.offset + kSlots * i], sizeof(LaunchDesc));
        d.reserved = stage;
        ops.push_back(d);
      }
      ++stage;
    }
    return ops;
  }

  // Whether the reduction `ref` may run after the operations `ops` of stages
  // >= from_stage instead of before them: none of them touches its destination
  // and none writes one of its sources.
  bool reduction_may_follow(Pass pass, const LaunchRef& ref, const std::vector<LaunchDesc>& ops,
                            int from_stage) const {
    const Plan& plan = plans_[pass][static_cast<size_t>(ref.plan)];
    const Launch& l = plan.launches[ref.index];
    const size_t bytes = l.key.n * (l.key.dtype == GINN_HIP_F32 ? 4 : 2);
    const uintptr_t d0 = reinterpret_cast<uintptr_t>(l.reduce_dst), d1 = d0 + bytes;
    uintptr_t s_lo = ~uintptr_t(0), s_hi = 0;
    for (size_t i = 0; i < l.count; ++i) {
      const uintptr_t b = reinterpret_cast<uintptr_t>(plan.blob[l.offset + i]);
      s_lo = std::min(s_lo, b);
      s_hi = std::max(s_hi, b + bytes);
    }
    auto overlaps = [](uintptr_t a0, uintptr_t a1, uintptr_t b0, uintptr_t b1) { return a0 < b1 && b0 < a1; };
    for (const LaunchDesc& d : ops) {
      if (d.reserved < from_stage || d.n == 0) continue;
      const size_t ob = d.n * (d.dtype == GINN_HIP_F32 ? 4 : 2);
      const uintptr_t w0 = reinterpret_cast<uintptr_t>(d.dst), w1 = w0 + ob;
      if (overlaps(w0, w1, d0, d1)) return false;
      for (const void* src : d.src)
        if (src && overlaps(reinterpret_cast<uintptr_t>(src), reinterpret_cast<uintptr_t>(src) + ob, d0, d1))
          return false;
      if (overlaps(w0, w1, s_lo, s_hi)) {  // near the sources: look at each
        for (size_t i = 0; i < l.count; ++i) {
          const uintptr_t b = reinterpret_cast<uintptr_t>(plan.blob[l.offset + i]);
          if (overlaps(w0, w1, b, b + bytes)) return false;
        }
      }
    }
    return true;
  }

  long build_chain(std::vector<LaunchDesc> ops, int stage) {
    if (stage < 2 || ops.empty() || ops.size() > 0x7fffffffu) return -1;
    struct Interval {
      uintptr_t begin, end;
      uint32_t op;
      bool write;
    };
    std::vector<Interval> ivs;
    ivs.reserve(ops.size() * 3);
    for (size_t i = 0; i < ops.size(); ++i) {
      const LaunchDesc& d = ops[i];
      const size_t bytes = d.n * (d.dtype == GINN_HIP_F32 ? 4 : 2);
      if (bytes == 0) continue;
      const uintptr_t w = reinterpret_cast<uintptr_t>(d.dst);
      ivs.push_back({w, w + bytes, static_cast<uint32_t>(i), true});
      for (const void* src : d.src)
        if (src) {
          const uintptr_t r = reinterpret_cast<uintptr_t>(src);
          ivs.push_back({r, r + bytes, static_cast<uint32_t>(i), false});
        }
    }
    std::sort(ivs.begin(), ivs.end(), [](const Interval& a, const Interval& b) { return a.begin < b.begin; });
    std::vector<uint32_t> parent(ops.size());
    for (size_t i = 0; i < parent.size(); ++i) parent[i] = static_cast<uint32_t>(i);
    auto find = [&](uint32_t x) {
      while (parent[x] != x) x = parent[x] = parent[parent[x]];
      return x;
    };
    auto join = [&](uint32_t a, uint32_t b) {
      a = find(a);
      b = find(b);
      if (a != b) parent[std::max(a, b)] = std::min(a, b);
    };
    // Sweep over the addresses with the intervals that are still open; a write
    // is joined with every open interval, a read with every open write.
    std::vector<Interval> open_w, open_r;
    auto prune = [](std::vector<Interval>& v, uintptr_t at) {
      size_t keep = 0;
      for (size_t i = 0; i < v.size(); ++i)
        if (v[i].end > at) v[keep++] = v[i];
      v.resize(keep);
    };
    for (const Interval& iv : ivs) {
      prune(open_w, iv.begin);
      prune(open_r, iv.begin);
      for (const Interval& o : open_w) join(iv.op, o.op);
      if (iv.write) {
        for (const Interval& o : open_r) join(iv.op, o.op);
        open_w.push_back(iv);
      } else {
        open_r.push_back(iv);
      }
    }
    // Order: by chain, inside a chain by stage, then as described.
    std::vector<uint32_t> order(ops.size());
    for (size_t i = 0; i < order.size(); ++i) order[i] = static_cast<uint32_t>(i);
    std::vector<uint32_t> root(ops.size());
    for (size_t i = 0; i < root.size(); ++i) root[i] = find(static_cast<uint32_t>(i));
    std::stable_sort(order.begin(), order.end(), [&](uint32_t a, uint32_t b) {
      if (root[a] != root[b]) return root[a] < root[b];
      return ops[a].reserved < ops[b].reserved;
    });
    std::vector<ginn_hip_chain_range> ranges;
    size_t work = 0;
    for (size_t i = 0; i < order.size(); ++i) {
      if (i == 0 || root[order[i]] != root[order[i - 1]]) {
        ranges.push_back({static_cast<unsigned>(i), 0u});
        work = 0;
      }
      ++ranges.back().count;
      work += ops[order[i]].n;
      if (work > kChainWork) return -1;
    }
    // One allocation: ranges (padded to the record size), then records.
    const size_t range_bytes = (ranges.size() * sizeof(ginn_hip_chain_range) + 63) / 64 * 64;
    std::vector<unsigned char> host(range_bytes + ops.size() * sizeof(LaunchDesc));
    std::memcpy(host.data(), ranges.data(), ranges.size() * sizeof(ginn_hip_chain_range));
    for (size_t i = 0; i < order.size(); ++i)
      std::memcpy(host.data() + range_bytes + i * sizeof(LaunchDesc), &ops[order[i]], sizeof(LaunchDesc));
    Chain c;
    c.dev = dev_->alloc(host.size());
    c.chains = ranges.size();
    c.ops = ops.size();
    c.stages = static_cast<size_t>(stage);
    GINN_HIP_CALL(ginn_hip_memcpy_h2d(ctx_, c.dev, host.data(), host.size()));
    GINN_HIP_CALL(ginn_hip_sync(ctx_));  // `host` goes away
    chains_.push_back(c);
    return static_cast<long>(chains_.size() - 1);
  }

  void launch_chain(const Chain& c) {
    const size_t range_bytes = (c.chains * sizeof(ginn_hip_chain_range) + 63) / 64 * 64;
    GINN_HIP_CALL(ginn_hip_multi_chain(
        ctx_, static_cast<int>(c.chains), static_cast<const ginn_hip_chain_range*>(c.dev),
        reinterpret_cast<const ginn_hip_multi_op*>(static_cast<const unsigned char*>(c.dev) + range_bytes)));
    ++launches_;
  }

  void fuse_pass(Pass pass) {
    auto& items = fused_[pass];
    items.clear();
    auto emit_launch = [&](const LaunchRef& ref) {
      if (!items.empty() && items.back().direct.empty() && items.back().plan == ref.plan &&
          items.back().first + items.back().count == ref.index) {
        ++items.back().count;  // next launch of the same plan
        return;
      }
      Item it;
      it.plan = ref.plan;
      it.first = ref.index;
      it.count = 1;
      items.push_back(std::move(it));
    };
    // The run under way: mixed launches in order, and reductions met on the
    // way with the number of mixed launches that came before each.
    std::vector<LaunchRef> run;
    std::vector<std::pair<LaunchRef, int>> reductions;
    // Mixed launches `part` as one chain followed by the reductions `reds`
    // (all of which may follow it), or every launch where it was recorded.
    auto emit_part = [&](const std::vector<LaunchRef>& part, const std::vector<std::pair<LaunchRef, int>>& reds) {
      const long chain =
          part.size() >= 2 ? build_chain(records_of(pass, part), static_cast<int>(part.size())) : -1;
      if (chain >= 0) {
        Item it;
        it.chain = chain;
        items.push_back(std::move(it));
        for (auto& r : reds) emit_launch(r.first);
        return;
      }
      size_t next = 0;
      for (size_t i = 0; i <= part.size(); ++i) {
        while (next < reds.size() && reds[next].second == static_cast<int>(i)) emit_launch(reds[next++].first);
        if (i < part.size()) emit_launch(part[i]);
      }
    };
    auto end_run = [&] {
      // A reduction that later operations of the run depend on stays where it
      // is and cuts the run in two.
      while (!run.empty() || !reductions.empty()) {
        const std::vector<LaunchDesc> ops = records_of(pass, run);
        size_t stuck = reductions.size();
        for (size_t k = 0; k < reductions.size() && stuck == reductions.size(); ++k)
          if (!reduction_may_follow(pass, reductions[k].first, ops, reductions[k].second)) stuck = k;
        if (stuck == reductions.size()) {
          emit_part(run, reductions);
          break;
        }
        const int cut = reductions[stuck].second;
        emit_part(std::vector<LaunchRef>(run.begin(), run.begin() + cut),
                  std::vector<std::pair<LaunchRef, int>>(reductions.begin(), reductions.begin() + stuck));
        emit_launch(reductions[stuck].first);
        run.erase(run.begin(), run.begin() + cut);
        reductions.erase(reductions.begin(), reductions.begin() + stuck + 1);
        for (auto& r : reductions) r.second -= cut;
      }
      run.clear();
      reductions.clear();
    };
    for (const Step& step : steps_[pass]) {
      if (!step.direct.empty()) {  // they run before the step's own plan
        end_run();
        Item it;
        it.direct = step.direct;
        items.push_back(std::move(it));
      }
      if (step.plan < 0) continue;
      const Plan& plan = plans_[pass][static_cast<size_t>(step.plan)];
      for (size_t li = 0; li < plan.launches.size(); ++li) {
        const Launch& l = plan.launches[li];
        const LaunchRef ref{step.plan, li};
        if (pass == kReset || l.zero_max) {
          end_run();
          emit_launch(ref);
        } else if (l.reduce_dst) {
          if (!l.late) reductions.emplace_back(ref, static_cast<int>(run.size()));
        } else {
          run.push_back(ref);
        }
      }
    }
    end_run();
  }

  void run_fused(Pass pass) {
    for (const Item& it : fused_[pass]) {
      for (BaseNode* n : it.direct) {
        if (pass == kForward) {
          n->forwarded = false;
          n->forward();
          settle_if_replayed_reader(n);
        } else if (pass == kReset) {
          n->reset_grad();
        } else {
          n->backward();
        }
      }
      if (it.plan >= 0) launch(plans_[pass][static_cast<size_t>(it.plan)], it.first, it.count);
      if (it.chain >= 0) launch_chain(chains_[static_cast<size_t>(it.chain)]);
    }
  }

  // freeze(): which nodes with a postponed value are read by a node that does not run itself in the frozen
  // forward pass (its work is replayed from the recording, so it never calls value()).
  void find_replayed_readers() {
    settle_after_forward_.clear();
    std::unordered_set<const BaseNode*> runs_itself;
    for (const Step& step : steps_[kForward])
      for (BaseNode* n : step.direct) runs_itself.insert(n);
    for (auto& n : list_) {
      if (runs_itself.count(n.get())) continue;
      for (auto& in : n->ins())
        if (dynamic_cast<PostponedValue*>(in.get())) settle_after_forward_.insert(in.get());
    }
  }
  void settle_if_replayed_reader(BaseNode* n) {
    if (!settle_after_forward_.empty() && settle_after_forward_.count(n))
      dynamic_cast<PostponedValue*>(n)->settle_value();
  }

  void seed_sink(double loss_coeff) {
    BaseNodePtr sink = list_.back();
    if (auto s = dynamic_ptr_cast<Node<Real>>(sink)) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(static_cast<Real>(loss_coeff));
    } else if (auto s = dynamic_ptr_cast<Node<Half>>(sink)) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(Half(static_cast<float>(loss_coeff)));
    } else if (auto s = dynamic_ptr_cast<Node<BFloat16>>(sink)) {
      GINN_ASSERT(s->has_grad());
      s->grad().fill(BFloat16(static_cast<float>(loss_coeff)));
    } else {
      GINN_THROW("Unexpected scalar type in sink node!");
    }
  }

 public:
  // The executor keeps the node handles of g alive; nodes must live on one GPU.
  explicit LevelExecutor(const Graph& g) : list_(g.nodes()) {
    GINN_ASSERT(!list_.empty());
    for (auto& n : list_)
      if (n->dev() && n->dev()->kind() == GPU) dev_ = n->dev();
    GINN_ASSERT(static_cast<bool>(dev_), "LevelExecutor: no node of the graph lives on a GPU");
    ctx_ = hip_ctx(static_cast<int>(dev_->id().idx));
    for (auto& n : list_)
      if (auto* p = dynamic_cast<PendingInPlace*>(n.get())) pending_steps_.push_back(p);
    build_levels();
  }
  LevelExecutor(const LevelExecutor&) = delete;
  LevelExecutor& operator=(const LevelExecutor&) = delete;
  ~LevelExecutor() {
    drop_graph();
    drop_chains();
    drop_late_reductions();
    for (auto& pass : plans_)
      for (auto& plan : pass)
        if (plan.dev) {
          try {
            dev_->free(plan.dev);
          } catch (...) {
          }
        }
  }

  // freeze(): the caller promises that, until thaw(), the graph is run again
  // and again unchanged -- no node rewired, resized, moved to other storage or
  // switched between has_grad states.  The passes then replay what the last
  // full pass of each kind recorded (the nodes that ran themselves and the
  // launch plans) without asking the other nodes anything.  Each of forward(),
  // reset_grad() and backward() must have run once before.
  LevelExecutor& freeze() {
    for (auto& steps : steps_) GINN_ASSERT(!steps.empty(), "LevelExecutor::freeze() before a full pass");
    GINN_ASSERT(!unplanned_fill_,
                "LevelExecutor::freeze(): a node that declares GradUse::Overwrites added to a gradient that "
                "reset_grad() had only flagged; run with set_lazy_grad_reset(false)");
    plan_late_reductions();
    find_replayed_readers();
    frozen_ = true;
    return *this;
  }
  LevelExecutor& thaw() {
    frozen_ = false;
    drop_graph();
    drop_chains();
    drop_late_reductions();
    return *this;
  }
  // fuse(): on a frozen executor, joins the table launches of consecutive
  // levels into one launch wherever no node runs itself between them: the
  // operations are regrouped into chains that do not touch each other's
  // memory (one per sequence for a recurrent cell unrolled over a minibatch),
  // each chain runs in one workgroup, level after level.  Same operations on
  // the same memory in the same order per element, hence the same results.
  // Runs of levels whose chains would be long stay as they are.
  LevelExecutor& fuse() {
    GINN_ASSERT(frozen_, "LevelExecutor::fuse() needs a frozen executor");
    drop_graph();
    drop_chains();
    fuse_pass(kForward);
    fuse_pass(kReset);
    fuse_pass(kBackward);
    fused_ready_ = true;
    return *this;
  }
  bool fused() const { return fused_ready_; }
  size_t chains() const { return chains_.size(); }
  bool frozen() const { return frozen_; }

  // record_pass(): records one frozen training pass -- forward(), reset_grad(),
  // backward(loss_coeff) -- as a device graph instead of running it (values and
  // gradients are NOT updated by this call); replay_pass() then launches the
  // whole pass with one call.  The promise of freeze() holds for the recording
  // as well; thaw() drops it.  Nodes of the graph must not wait for the device
  // or copy to or from the host while they run (none of this library's do).
  LevelExecutor& record_pass(double loss_coeff = 1) {
    GINN_ASSERT(frozen_, "LevelExecutor::record_pass() needs a frozen executor");
    drop_graph();
    GINN_HIP_CALL(ginn_hip_capture_begin(ctx_));
    try {
      forward();
      reset_grad();
      backward(loss_coeff);
    } catch (...) {
      ginn_hip_graph* broken = nullptr;
      ginn_hip_capture_end(ctx_, &broken);
      if (broken) ginn_hip_graph_destroy(broken);
      throw;
    }
    GINN_HIP_CALL(ginn_hip_capture_end(ctx_, &pass_graph_));
    return *this;
  }
  LevelExecutor& replay_pass() {
    GINN_ASSERT(pass_graph_ != nullptr, "LevelExecutor::replay_pass() before record_pass()");
    GINN_HIP_CALL(ginn_hip_graph_launch(pass_graph_));
    return *this;
  }
  bool recorded() const { return pass_graph_ != nullptr; }
  // Kernel launches in the recorded pass (0 before record_pass()).
  size_t recorded_kernels() const {
    size_t n = 0;
    if (pass_graph_) GINN_HIP_CALL(ginn_hip_graph_kernel_count(pass_graph_, &n));
    return n;
  }

  LevelExecutor& reset_forwarded() {
    if (frozen_) return *this;  // forward() re-runs what it has to
    for (auto& n : list_) n->reset_forwarded();
    return *this;
  }

  // An in-place step that nobody has asked for by the end of the pass runs
  // then (PendingInPlace), as at the end of Graph::forward().
  LevelExecutor& forward() {
    if (frozen_ && fused_ready_) {
      run_fused(kForward);
      for (PendingInPlace* p : pending_steps_) p->settle();
      return *this;
    }
    if (frozen_) {
      for (Step& step : steps_[kForward]) {
        for (BaseNode* n : step.direct) {
          n->forwarded = false;
          n->forward();
          settle_if_replayed_reader(n);
        }
        if (step.plan >= 0) launch(plans_[kForward][static_cast<size_t>(step.plan)]);
      }
      for (PendingInPlace* p : pending_steps_) p->settle();
      return *this;
    }
    cursor_ = 0;
    descs_.clear();
    for (size_t li = 0; li < levels_.size(); ++li) {
      Step& step = begin_step(kForward, li);
      for (BaseNode* n : levels_[li]) {
        if (n->forwarded) continue;
        if (n->describe_forward(descs_)) {
          n->forwarded = true;
        } else {
          n->forward();
          step.direct.push_back(n);
        }
      }
      flush(kForward, step);
    }
    for (PendingInPlace* p : pending_steps_) p->settle();
    return *this;
  }

  LevelExecutor& reset_grad() {
    if (frozen_ && fused_ready_) {
      for (BaseNode* n : lazy_direct_) n->reset_grad_lazy();
      run_fused(kReset);
      return *this;
    }
    if (frozen_) {
      for (BaseNode* n : lazy_direct_) n->reset_grad_lazy();
      for (Step& step : steps_[kReset]) {
        for (BaseNode* n : step.direct) n->reset_grad();
        if (step.plan >= 0) launch(plans_[kReset][static_cast<size_t>(step.plan)]);
      }
      return *this;
    }
    cursor_ = 0;
    descs_.clear();
    lazy_.clear();
    const std::vector<unsigned char> lazy = lazy_grad_candidates(list_, id_);
    Step& step = begin_step(kReset, 0);
    for (size_t i = 0; i < list_.size(); ++i) {  // graph order: views map onto gradients sized before them
      BaseNode* n = list_[i].get();
      if (lazy[i]) {
        n->reset_grad_lazy();
        lazy_.push_back(n);
      } else if (!n->describe_reset_grad(descs_)) {
        n->reset_grad();
        step.direct.push_back(n);
      }
    }
    flush(kReset, step);
    return *this;
  }

  // Seeds the sink gradient with loss_coeff and back-propagates level by
  // level; reset_grad() must have run (ginn/node.h:237-254).
  LevelExecutor& backward(double loss_coeff = 1) {
    seed_sink(loss_coeff);
    internal::FoldWindow folds(id_);  // row sums into leaf gradients are folded once, at the end
    if (frozen_) {
      if (fused_ready_) {
        run_fused(kBackward);
      } else {
        for (Step& step : steps_[kBackward]) {
          for (BaseNode* n : step.direct) n->backward();
          if (step.plan >= 0) launch(plans_[kBackward][static_cast<size_t>(step.plan)]);
        }
      }
      for (BaseNode* n : lazy_direct_) n->clear_lazy_zero();  // all taken already, unless a node returned early
      run_late_reductions();
      folds.close();
      return *this;
    }
    cursor_ = 0;
    descs_.clear();
    unplanned_fill_ = false;
    taken_by_plans_.clear();
    struct LogGuard {
      ~LogGuard() { internal::lazy_take_log() = nullptr; }
    } guard;
    for (size_t k = 0; k < levels_.size(); ++k) {
      Step& step = begin_step(kBackward, k);
      for (BaseNode* n : levels_[levels_.size() - 1 - k]) {
        if (!n->has_grad()) continue;
        const size_t fills = internal::lazy_grad_settles();
        internal::lazy_take_log() = &taken_by_plans_;
        const bool described = n->describe_backward(descs_);
        internal::lazy_take_log() = nullptr;
        if (!described) {
          n->backward();
          step.direct.push_back(n);
        } else if (internal::lazy_grad_settles() != fills) {
          unplanned_fill_ = true;
        }
      }
      flush(kBackward, step);
    }
    folds.close();
    std::sort(taken_by_plans_.begin(), taken_by_plans_.end());
    lazy_direct_.clear();
    for (BaseNode* n : lazy_)
      if (!std::binary_search(taken_by_plans_.begin(), taken_by_plans_.end(), n)) lazy_direct_.push_back(n);
    return *this;
  }

  size_t levels() const { return levels_.size(); }
  // Table launches issued and node operations they covered since construction.
  size_t launches() const { return launches_; }
  size_t described() const { return described_; }
  // Flushes whose plan had to be (re)built: the first pass, or changed shapes / storage.
  size_t rebuilt() const { return rebuilt_; }
};

}  // namespace ginn

#endif  // GINN_LEVEL_EXEC_H
