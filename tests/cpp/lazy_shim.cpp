// Test shim for gradients that reset_grad() flags instead of zeroing
// (BaseNode::GradUse in ginn_amd/ginn/node.h): one graph in which every node
// that can overwrite is the only user of its input at least once, run with
// the flagging on and off, node by node and through the level executor in all
// of its modes.  The reference zeroes every gradient (ginn/node.h:218-222) and
// adds in every backward; both runs must give the same gradients.
#include <cmath>
#include <limits>
#include <string>
#include <vector>

#include <ginn/ginn.h>

using namespace ginn;

namespace {

thread_local std::string g_error;

template <typename S>
Ptr<DataNode<S>> data_of(const Shape& shape, const float* vals, bool has_grad) {
  auto x = Data<S>(cpu(), shape);
  S* p = x->value().v();
  for (Size i = 0; i < x->value().size(); ++i) p[i] = S(vals[i]);
  x->move_to(gpu());
  x->set_has_grad(has_grad);
  return x;
}

template <typename S>
Ptr<WeightNode<S>> weight_of(const Shape& shape, const float* vals) {
  auto w = Weight<S>(cpu(), shape);
  S* p = w->value().v();
  for (Size i = 0; i < w->value().size(); ++i) p[i] = S(vals[i]);
  w->move_to(gpu());
  return w;
}

template <typename S>
void read_back(const Tensor<S>& t, float* out) {
  const auto v = t.vector();
  for (size_t i = 0; i < v.size(); ++i) out[i] = static_cast<float>(v[i]);
}

// A small attention block followed by a gated product and a vocabulary head.
// C = hs * nh channels, B sequences of T positions, V classes.  params:
//   0 Wk [C,C]  1 bk [C]  2 Wq [C,C]  3 bq [C]  4 Wv [C,C]  5 bv [C]
//   6 Wp [C,C]  7 Wg [C,C]  8 Wh [V,C]  9 bh [V]
// mode: 0 = Graph; 1 = executor, every pass planned anew; 2 = frozen; 3 = frozen
// and chained; 4 = recorded as a device graph.  `passes` passes are run; the
// gradients of the last one are returned: dx, then the ten parameters.
template <typename S>
int lazy_graph(int mode, int passes, int hs, int nh, int B, int T, int V, const float* x, const int* targets,
               const float* const* params, float* out_loss, float* out_dx, float* const* out_grads,
               long* out_flagged, long* out_fills) {
  const Size C = static_cast<Size>(hs) * nh;
  const Shape shapes[10] = {{C, C}, {C}, {C, C}, {C}, {C, C}, {C}, {C, C}, {C, C}, {V, C}, {V}};
  std::vector<Ptr<WeightNode<S>>> w;
  for (int i = 0; i < 10; ++i) w.push_back(weight_of<S>(shapes[i], params[i]));
  enum { Wk, bk, Wq, bq, Wv, bv, Wp, Wg, Wh, bh };

  auto X = data_of<S>({C, B, T}, x, true);
  auto Y = Data<Int>(cpu(), Shape{B * T});
  for (int i = 0; i < B * T; ++i) Y->value().v()[i] = targets[i];
  Y->move_to(gpu());
  Y->set_has_grad(false);

  auto heads = [&](const NodePtr<S>& t, Shape perm) -> NodePtr<S> {
    return Permute(NodePtr<S>(Reshape(t, Shape{hs, nh, B, T})), std::move(perm));
  };
  NodePtr<S> a = LayerNorm(NodePtr<S>(X));                                // X: two users (here and the residual)
  auto k = heads(Affine(w[Wk], a, w[bk]), {3, 0, 2, 1});                  // T, hs, B, nh
  auto q = heads(Affine<TanhOp>(w[Wq], a, w[bq]), {0, 3, 2, 1});          // hs, T, B, nh
  auto v = heads(Affine(w[Wv], a, w[bv]), {0, 3, 2, 1});
  NodePtr<S> att = InPlaceProdScalar(NodePtr<S>(BatchedProd(k, q)), 1.f / std::sqrt(static_cast<float>(hs)));
  NodePtr<S> mask = Reshape(NodePtr<S>(UpperTri<S>(gpu(), static_cast<Size>(T))), Shape{T, T, 1, 1});
  att = InPlaceMask(att, mask, -std::numeric_limits<float>::infinity());
  att = Softmax(att);
  NodePtr<S> y = BatchedProd(v, att);                                      // hs, T, B, nh
  y = Permute(y, Shape{0, 3, 2, 1});                                       // hs, nh, B, T
  NodePtr<S> flat = Reshape(y, Shape{C, B * T});
  NodePtr<S> proj = Prod(NodePtr<S>(w[Wp]), flat);                         // plain product, no bias
  NodePtr<S> gate = Sigmoid(NodePtr<S>(Prod(NodePtr<S>(w[Wg]), NodePtr<S>(Reshape(NodePtr<S>(X), Shape{C, B * T})))));
  NodePtr<S> mixed = CwiseProd(proj, gate);                                // both operands have one user
  NodePtr<S> scaled = ProdScalar(NodePtr<S>(Tanh(mixed)), 0.5);
  NodePtr<S> sum = Add(scaled, NodePtr<S>(Reshape(NodePtr<S>(LayerNorm(NodePtr<S>(Map(scaled)))), Shape{C, B * T})));
  auto logits = Affine(w[Wh], sum, w[bh]);
  auto loss = Mean(NodePtr<S>(PickNegLogSoftmax(NodePtr<S>(logits), Y)));

  Graph g(loss);
  const std::vector<unsigned char> lazy = lazy_grad_candidates(g.nodes());
  long flagged = 0;
  for (unsigned char f : lazy) flagged += f;
  if (out_flagged) *out_flagged = flagged;

  auto pass = [&](auto& runner) {
    runner.reset_forwarded();
    runner.forward();
    runner.reset_grad();
    runner.backward(1.);
  };
  const size_t fills_before = internal::lazy_grad_settles();
  if (mode == 0) {
    for (int i = 0; i < passes; ++i) pass(g);
  } else {
    LevelExecutor ex(g);
    pass(ex);
    if (mode >= 2) ex.freeze();
    if (mode == 3) ex.fuse();
    if (mode == 4) {
      ex.record_pass();
      for (int i = 1; i < passes; ++i) ex.replay_pass();
    } else {
      for (int i = 1; i < passes; ++i) pass(ex);
    }
  }
  gpu()->synchronize();
  if (out_fills) *out_fills = static_cast<long>(internal::lazy_grad_settles() - fills_before);
  read_back(loss->value(), out_loss);
  read_back(X->grad(), out_dx);
  for (int i = 0; i < 10; ++i) read_back(w[i]->grad(), out_grads[i]);
  return 0;
}

// Batched products on permuted views (node/slices.h): X [C x B T] is projected three times (Prod with Wk, Wq,
// Wv [C x C], C = hs nh), each projection reshaped to [hs, nh, B, T] and permuted to the slices of a head
// (k: [T, hs, B, nh], q and v: [hs, T, B, nh]); s = BatchedProd(k, q), y = BatchedProd(v, s), y permuted back to
// [hs, nh, B, T] and reshaped to [C x B T]; loss = Sum(mask (*) y).  Pass 1 runs on x1, then x2 is written into
// the SAME input tensor and pass 2 runs (a frozen executor replays; a value that was postponed and never asked
// for would show up as pass 1's).  mode: 0 = Graph, 1 = executor, 2 = frozen executor, 3 = frozen and recorded
// as a device graph.  read: 1 = the values of k and of s are read back between forward and backward of pass 2
// (the postponed copy / product must then run, and everything still agree).  Outputs of pass 2: y, dX, dWk,
// dWq, dWv; *out_kernels: kernel launches of the recorded pass (mode 3).
template <typename S>
int permuted_products(int mode, int read, int hs, int nh, int B, int T, const float* x1, const float* x2,
                      const float* const* w, const float* mask, float* out_y, float* out_dx, float* const* out_dw,
                      float* out_k, float* out_s, long* out_kernels) {
  const Size C = static_cast<Size>(hs) * nh, N = static_cast<Size>(B) * T;
  auto X = data_of<S>({C, N}, x1, true);
  std::vector<Ptr<WeightNode<S>>> W;
  for (int i = 0; i < 3; ++i) W.push_back(weight_of<S>({C, C}, w[i]));
  auto M = data_of<S>({C, N}, mask, false);
  auto heads = [&](int i, Shape perm) -> NodePtr<S> {
    NodePtr<S> proj = Prod(NodePtr<S>(W[i]), NodePtr<S>(X));
    return Permute(NodePtr<S>(Reshape(proj, Shape{hs, nh, B, T})), std::move(perm));
  };
  NodePtr<S> k = heads(0, {3, 0, 2, 1}), q = heads(1, {0, 3, 2, 1}), v = heads(2, {0, 3, 2, 1});
  NodePtr<S> s = BatchedProd(k, q);
  NodePtr<S> y = Permute(NodePtr<S>(BatchedProd(v, s)), Shape{0, 3, 2, 1});
  NodePtr<S> flat = Reshape(y, Shape{C, N});
  auto loss = Sum(CwiseProd(flat, NodePtr<S>(M)));
  Graph g(loss);
  auto set_input = [&](const float* vals) {
    Tensor<S> host(cpu(), X->value().shape());
    for (Size i = 0; i < host.size(); ++i) host.v()[i] = S(vals[i]);
    X->value() = host.copy_to(gpu());  // same size: copies into the tensor's storage
  };
  auto pass = [&](auto& runner, bool look) {
    runner.reset_forwarded();
    runner.forward();
    if (look) {
      read_back(k->value(), out_k);
      read_back(s->value(), out_s);
    }
    runner.reset_grad();
    runner.backward(1.);
  };
  if (mode == 0) {
    pass(g, false);
    set_input(x2);
    pass(g, read != 0);
  } else {
    LevelExecutor ex(g);
    pass(ex, false);
    if (mode >= 2) ex.freeze();
    set_input(x2);
    if (mode == 3) {
      ex.record_pass();
      if (out_kernels) *out_kernels = static_cast<long>(ex.recorded_kernels());
      ex.replay_pass();
      if (read) {
        read_back(k->value(), out_k);
        read_back(s->value(), out_s);
      }
    } else {
      pass(ex, read != 0);
    }
  }
  gpu()->synchronize();
  read_back(flat->value(), out_y);
  read_back(X->grad(), out_dx);
  for (int i = 0; i < 3; ++i) read_back(W[i]->grad(), out_dw[i]);
  return 0;
}

}  // namespace

#define DISPATCH(DTYPE, CALL)                                     \
  try {                                                           \
    switch (DTYPE) {                                              \
      case GINN_HIP_F32: { using S = Real; return CALL; }         \
      case GINN_HIP_F16: { using S = Half; return CALL; }         \
      case GINN_HIP_BF16: { using S = BFloat16; return CALL; }    \
    }                                                             \
    g_error = "unknown dtype";                                    \
    return 1;                                                     \
  } catch (const std::exception& e) {                             \
    g_error = e.what();                                           \
    return 2;                                                     \
  }

extern "C" {

const char* lazy_last_error() { return g_error.c_str(); }

// lazy != 0: reset_grad() may flag gradients (the default of the library).
int shim_lazy_graph(int dtype, int lazy, int mode, int passes, int hs, int nh, int B, int T, int V, const float* x,
                    const int* targets, const float* const* params, float* out_loss, float* out_dx,
                    float* const* out_grads, long* out_flagged, long* out_fills) {
  struct Restore {
    bool was = lazy_grad_reset();
    ~Restore() { set_lazy_grad_reset(was); }
  } restore;
  set_lazy_grad_reset(lazy != 0);
  DISPATCH(dtype, (lazy_graph<S>(mode, passes, hs, nh, B, T, V, x, targets, params, out_loss, out_dx, out_grads,
                                 out_flagged, out_fills)));
}

// Products into weight gradients on the second stream of the GPU (on by default) or on the one stream.
void shim_set_beside_pass(int on) { set_beside_pass(on != 0); }

// A weight with several gradient writers in one pass: W [d x d] is the left operand of a product of
// 2 d^3 flops (large enough for the second stream when d >= 800), of a narrow product W x2 (always on
// the pass's stream) and an operand of an Add; V [d x d] has the large product as its only user.
// Three passes; out_dw / out_dv: the gradients of W and V after the last one.  out_beside: launches
// that went to the second stream.  mode: 0 = Graph, 1 = executor, 2 = frozen executor.
int shim_permuted_products(int dtype, int mode, int read, int hs, int nh, int B, int T, const float* x1, const float* x2,
                           const float* const* w, const float* mask, float* out_y, float* out_dx,
                           float* const* out_dw, float* out_k, float* out_s, long* out_kernels) {
  try {
    switch (dtype) {
      case GINN_HIP_F32:
        return permuted_products<Real>(mode, read, hs, nh, B, T, x1, x2, w, mask, out_y, out_dx, out_dw, out_k, out_s,
                                       out_kernels);
      case GINN_HIP_F16:
        return permuted_products<Half>(mode, read, hs, nh, B, T, x1, x2, w, mask, out_y, out_dx, out_dw, out_k, out_s,
                                       out_kernels);
      case GINN_HIP_BF16:
        return permuted_products<BFloat16>(mode, read, hs, nh, B, T, x1, x2, w, mask, out_y, out_dx, out_dw, out_k,
                                           out_s, out_kernels);
    }
    g_error = "unknown dtype";
    return 1;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 2;
  }
}

int shim_shared_weight_graph(int mode, int d, const float* w, const float* v, const float* x1, const float* x2,
                             float* out_loss, float* out_dw, float* out_dv, long* out_beside) {
  try {
    const Size n = d;
    auto W = weight_of<Real>({n, n}, w);
    auto V = weight_of<Real>({n, n}, v);
    auto X1 = data_of<Real>({n, n}, x1, false);
    auto X2 = data_of<Real>({n, 8}, x2, false);
    NodePtr<Real> big = Prod(NodePtr<Real>(W), NodePtr<Real>(X1));      // dW += d(big) X1^T: 2 d^3 flops
    NodePtr<Real> alone = Prod(NodePtr<Real>(V), NodePtr<Real>(big));   // V's only user; also 2 d^3 flops
    NodePtr<Real> small = Prod(NodePtr<Real>(W), NodePtr<Real>(X2));    // dW += d(small) X2^T
    NodePtr<Real> added = Add(NodePtr<Real>(W), NodePtr<Real>(Tanh(alone)));  // dW += d(added)
    auto loss = Add(NodePtr<Real>(Sum(NodePtr<Real>(Tanh(added)))), NodePtr<Real>(Sum(NodePtr<Real>(Sigmoid(small)))));
    Graph g(loss);
    auto pass = [&](auto& runner) {
      runner.reset_forwarded();
      runner.forward();
      runner.reset_grad();
      runner.backward(1.);
    };
    const size_t before = internal::beside_launches();
    if (mode == 0) {
      for (int i = 0; i < 3; ++i) pass(g);
    } else {
      LevelExecutor ex(g);
      pass(ex);
      if (mode == 2) ex.freeze();
      for (int i = 1; i < 3; ++i) pass(ex);
    }
    gpu()->synchronize();
    if (out_beside) *out_beside = static_cast<long>(internal::beside_launches() - before);
    read_back(loss->value(), out_loss);
    read_back(W->grad(), out_dw);
    read_back(V->grad(), out_dv);
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 2;
  }
}

// In-place steps that postpone their work (InPlaceProdScalar, InPlaceMask; ginn/node/inplace.h:104-123,
// 152-212 overwrite the input in forward()).  scores = A B [3 x 2], scaled by 0.5, entries with mask 0 set to -5.
// which: 0 = the mask step is the sink: nobody reads its value; 1 = a Softmax behind it takes the steps over;
// both: out = the SCORES node's own value after Graph::forward() (what a holder of the upstream node sees).
// 2, 3 = the same two through LevelExecutor::forward().
// 4 = a skip left over by a backward pass that was cut short: the Softmax's backward is run by hand on a
// flagged gradient (it does the two steps' backward itself and tells them to skip theirs), the steps' own
// backward never runs; the next pass, with flagging off, needs them.  out = d(scores) of that pass followed by
// d(scores) of the same pass on a fresh graph (6 + 6 values).
int shim_inplace_semantics(int which, const float* a, const float* b, const float* mask, float* out) {
  try {
    auto build = [&](bool softmax, NodePtr<Real>& scores, NodePtr<Real>& top) {
      auto A = data_of<Real>({3, 4}, a, true);
      auto B = data_of<Real>({4, 2}, b, true);
      auto M = data_of<Real>({3, 2}, mask, false);
      scores = Prod(NodePtr<Real>(A), NodePtr<Real>(B));
      NodePtr<Real> x = InPlaceProdScalar(scores, 0.5);
      x = InPlaceMask(x, NodePtr<Real>(M), -5.f);
      top = softmax ? NodePtr<Real>(Softmax(x)) : x;
    };
    NodePtr<Real> scores, top;
    if (which <= 3) {
      build(which % 2 == 1, scores, top);
      Graph g(top);
      if (which < 2) {
        g.forward();
      } else {
        LevelExecutor ex(g);
        ex.forward();
      }
      read_back(scores->value(), out);
      return 0;
    }
    if (which == 4) {
      struct Restore {
        bool was = lazy_grad_reset();
        ~Restore() { set_lazy_grad_reset(was); }
      } restore;
      for (int fresh = 0; fresh < 2; ++fresh) {
        build(true, scores, top);
        NodePtr<Real> loss = Sum(NodePtr<Real>(CwiseProd(top, top)));
        Graph g(loss);
        g.forward();
        if (!fresh) {
          set_lazy_grad_reset(true);
          g.reset_grad();               // flags d(scores): the Softmax is the chain's only user
          top->grad().fill(1.f);
          top->backward();              // fused backward; tells the two steps to skip theirs
        }
        set_lazy_grad_reset(false);
        g.reset_grad();
        g.backward(1.);
        read_back(scores->grad(), out + 6 * fresh);
      }
      return 0;
    }
    g_error = "unknown case";
    return 1;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 2;
  }
}

// What everybody but the one overwriting user sees of a flagged gradient.
// which: 0 = read between reset_grad() and backward(): zeros, not what the
// last pass left; 1 = two graphs that share a node, reset one after the other
// and run one after the other: the shared gradient is the sum; 2 = a node with
// two users is not flagged, one with a single accumulating user neither.
// out: [0] = the largest |value| read (case 0), the gradient of the shared
// node's first entry (case 1), the number of flagged nodes (case 2).
int shim_lazy_semantics(int which, float* out) {
  try {
    auto A = Data<Real>(gpu(), Shape{3, 4});
    auto B = Data<Real>(gpu(), Shape{4, 2});
    A->value().fill(0.5f);
    B->value().fill(2.f);
    if (which == 0) {
      auto P = Prod(A, B);
      auto loss = Sum(NodePtr<Real>(Tanh(NodePtr<Real>(P))));
      Graph g(loss);
      g.forward();
      g.reset_grad();
      g.backward(1.);
      g.reset_grad();  // A, B and P are flagged again and still hold the last pass's gradients
      float worst = 0.f;
      for (const auto* t : {&A->grad(), &B->grad(), &P->grad()})
        for (float v : t->vector()) worst = std::max(worst, std::fabs(v));
      out[0] = worst;
      return 0;
    }
    if (which == 1) {
      auto P = Prod(A, B);  // shared: one overwriting user in each graph
      auto l1 = Sum(NodePtr<Real>(Tanh(NodePtr<Real>(P))));
      auto l2 = Sum(NodePtr<Real>(ProdScalar(NodePtr<Real>(P), 3.0)));
      Graph g1(l1), g2(l2);
      g1.forward();
      g2.forward();
      g1.reset_grad();
      g2.reset_grad();
      g1.backward(1.);
      g2.backward(1.);
      // dA = (tanh'(4) + 3) * (ones[3,2] * B^T) from g1's pass over P plus g2's second pass over P's
      // accumulated gradient; what matters here is dP itself: tanh'(4) + 3.
      out[0] = P->grad().vector()[0];
      return 0;
    }
    if (which == 2) {
      auto P = Prod(A, B);                                       // two users below: zeroed
      auto S1 = Sum(NodePtr<Real>(P));                           // Sum adds to its input's gradient
      auto Q = CwiseProd(NodePtr<Real>(P), NodePtr<Real>(P));    // the same node twice: two uses
      auto loss = Add(NodePtr<Real>(S1), NodePtr<Real>(Sum(NodePtr<Real>(Q))));
      Graph g(loss);
      const auto lazy = lazy_grad_candidates(g.nodes());
      long n = 0;
      for (size_t i = 0; i < lazy.size(); ++i)
        if (lazy[i]) {
          ++n;
          if (g.nodes()[i].get() == static_cast<BaseNode*>(P.get())) n += 1000;  // must not happen
        }
      out[0] = static_cast<float>(n);
      return 0;
    }
    g_error = "unknown case";
    return 1;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 2;
  }
}

}  // extern "C"
