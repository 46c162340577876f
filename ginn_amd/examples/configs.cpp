// Whole graphs of the build target's configurations, built with the
// header-only host layer and run on gpu(); exported with a C interface so that
// the parity tests and the benchmark drive the same code.
//   * an MLP of AffineNodes closed by Sum(PickNegLogSoftmax)
//     (graph of examples/mnist.cu.cpp:127-137);
//   * the reference's own Autobatch equivalence cases (test/autobatch.cpp:72-190);
//   * LSTM gates over many ragged sequences, plain and through Autobatch
//     (recurrence of ginn/model/lstm.h:91-103 without peepholes, one fused
//     Affine per step).
// Every entry point returns 0, or non-zero with the message in scenario_last_error().
#include <chrono>
#include <cmath>
#include <cstring>
#include <limits>
#include <string>
#include <vector>

#include <functional>

#include <ginn/autobatch.h>
#include <ginn/ginn.h>
#include <ginn/level_exec.h>
#include <ginn/update/update.h>

using namespace ginn;

namespace {

thread_local std::string g_error;
// scenario_set_device(1): the scenarios keep their graphs on cpu() and run through the host layer's own
// loops (ginn/cpu_ops.h), node by node -- the same graph code as on the device, as a host baseline.
bool g_on_cpu = false;
DevPtr place() { return g_on_cpu ? DevPtr(cpu()) : DevPtr(gpu()); }

template <typename S>
void upload(Tensor<S>& t, const float* vals) {
  Tensor<S> host(cpu(), t.shape());
  S* p = host.v();
  for (Size i = 0; i < host.size(); ++i) p[i] = S(vals[i]);
  t = host.copy_to(t.dev());
}

template <typename S>
void read_back(const Tensor<S>& t, float* out) {
  if (!out) return;
  const auto v = t.vector();
  for (size_t i = 0; i < v.size(); ++i) out[i] = static_cast<float>(v[i]);
}

template <typename S>
Ptr<DataNode<S>> data_from(const Shape& shape, const float* vals, bool has_grad) {
  auto x = Data<S>(place(), shape);
  upload(x->value(), vals);
  x->set_has_grad(has_grad);
  return x;
}

template <typename S>
Ptr<WeightNode<S>> weight_from(const Shape& shape, const float* vals) {
  auto w = Weight<S>(place(), shape);
  upload(w->value(), vals);
  return w;
}

template <typename S>
std::unique_ptr<NonlinOp<S>> make_op(int act) {
  switch (act) {
    case GINN_HIP_ACT_IDENTITY: return std::make_unique<IdentityOp<S>>();
    case GINN_HIP_ACT_TANH: return std::make_unique<TanhOp<S>>();
    case GINN_HIP_ACT_RELU: return std::make_unique<ReluOp<S>>();
    case GINN_HIP_ACT_SIGMOID: return std::make_unique<SigmoidOp<S>>();
    case GINN_HIP_ACT_GELU: return std::make_unique<GeluOp<S>>();
    case GINN_HIP_ACT_GELU2: return std::make_unique<Gelu2Op<S>>();
  }
  GINN_THROW("unknown activation");
  return nullptr;
}

double now_ms() {
  using namespace std::chrono;
  return duration<double, std::milli>(steady_clock::now().time_since_epoch()).count();
}

// What follows backward() in every timed pass: the weight update of a training
// step when a scenario asks for one (scenario_set_training), nothing otherwise.
std::function<void()> g_after_backward;
int g_train_rule = -1;  // -1: no update, 0: Sgd, 1: Adam
float g_train_lr = 1e-3f, g_train_clip = 5.f;

template <typename S>
std::unique_ptr<Updater<S>> make_updater() {
  if (g_train_rule == 0) return std::make_unique<update::Sgd<S>>(g_train_lr, g_train_clip);
  if (g_train_rule == 1) return std::make_unique<update::Adam<S>>(g_train_lr, g_train_clip);
  return nullptr;
}

// One training-style pass, `iters` times: forward, reset_grad, backward(1).
// Returns the mean wall time per pass (device drained on both sides).
double run_passes(Graph& g, int iters) {
  if (!g_on_cpu) gpu()->synchronize();
  const double t0 = now_ms();
  for (int it = 0; it < iters; ++it) {
    g.reset_forwarded();
    g.forward();
    g.reset_grad();
    g.backward(1.);
    if (g_after_backward) g_after_backward();
  }
  if (!g_on_cpu) gpu()->synchronize();
  return (now_ms() - t0) / (iters > 0 ? iters : 1);
}

// `iters` replays of a recorded pass (one graph launch each).
double run_replays(LevelExecutor& ex, int iters) {
  gpu()->synchronize();
  const double t0 = now_ms();
  for (int it = 0; it < iters; ++it) {
    ex.replay_pass();
    if (g_after_backward) g_after_backward();
  }
  gpu()->synchronize();
  return (now_ms() - t0) / (iters > 0 ? iters : 1);
}

// The same passes through the level executor (element-wise nodes of equal
// height share launches).
double run_passes(LevelExecutor& ex, int iters) {
  gpu()->synchronize();
  const double t0 = now_ms();
  for (int it = 0; it < iters; ++it) {
    ex.reset_forwarded();
    ex.forward();
    ex.reset_grad();
    ex.backward(1.);
    if (g_after_backward) g_after_backward();
  }
  gpu()->synchronize();
  return (now_ms() - t0) / (iters > 0 ? iters : 1);
}

// How the static configurations (MLP, GPT layer) are run: 0 = Graph, node by
// node; bit 1 = through the level executor; bit 2 = frozen after its first
// pass; bit 3 = the frozen pass recorded as a device graph and replayed; bit 4 (with bit 2) = table launches
// of consecutive levels joined into chain launches.
int g_exec_mode = 0;

// Zero fills made on demand during the timed passes of the last run_warm(): a
// gradient that reset_grad() had only flagged was read or added to before its
// user overwrote it.  None are expected; each is a launch of its own.
long g_timed_fills = 0;
// Kernel launches of the pass last recorded as a device graph (forward, reset_grad, backward).
long g_recorded_kernels = 0;

struct FillCount {
  size_t before = internal::lazy_grad_settles();
  void start() { before = internal::lazy_grad_settles(); }
  ~FillCount() { g_timed_fills = static_cast<long>(internal::lazy_grad_settles() - before); }
};

// Warm-up pass (first-touch allocations, launch plans), then `iters` timed ones.
double run_warm(Graph& g, int iters) {
  FillCount count;
  if ((g_exec_mode & 2) && !g_on_cpu) {
    LevelExecutor ex(g);
    run_passes(ex, 1);
    if (g_exec_mode & 4) ex.freeze();
    if ((g_exec_mode & 20) == 20) ex.fuse();
    if ((g_exec_mode & 12) == 12) {
      ex.record_pass();
      g_recorded_kernels = static_cast<long>(ex.recorded_kernels());
      ex.replay_pass();  // the first replay also loads the graph onto the device
      count.start();
      return run_replays(ex, iters);
    }
    count.start();
    return run_passes(ex, iters);
  }
  run_passes(g, 1);
  count.start();
  return run_passes(g, iters);
}

template <typename S>
int mlp(int batch, int n_layers, const int* dims, const int* acts, const float* x, const int* labels,
        const float* const* W, const float* const* b, int iters, float* out_loss, float* out_nll,
        float* const* dW, float* const* db, float* out_ms) {
  auto X = data_from<S>({dims[0], batch}, x, false);
  auto Y = Data<Int>(cpu(), Shape{batch});
  for (int i = 0; i < batch; ++i) Y->value().v()[i] = labels[i];
  Y->move_to(place());
  Y->set_has_grad(false);

  std::vector<Ptr<WeightNode<S>>> Ws, bs;
  NodePtr<S> h = X;
  for (int l = 0; l < n_layers; ++l) {
    Ws.push_back(weight_from<S>({dims[l + 1], dims[l]}, W[l]));
    bs.push_back(weight_from<S>({dims[l + 1]}, b[l]));
    h = make_ptr<AffineNode<S>>(make_op<S>(acts[l]), std::vector<NodePtr<S>>{Ws[l], h, bs[l]});
  }
  auto nll = PickNegLogSoftmax(h, Y);
  auto loss = Sum(nll);
  Graph g(loss);
  const double ms = run_warm(g, iters);
  if (out_ms) *out_ms = static_cast<float>(ms);
  read_back(loss->value(), out_loss);
  read_back(nll->value(), out_nll);
  for (int l = 0; l < n_layers; ++l) {
    read_back(Ws[l]->grad(), dW[l]);
    read_back(bs[l]->grad(), db[l]);
  }
  return 0;
}

// The same MLP trained for `steps` steps on one batch, the loop of the reference's
// examples (examples/mnist.cu.cpp:127-141: forward, reset_grad, backward, updater.update(g)).
// rule: 0 = Sgd, 1 = Adam; together != 0: update(graph), all weights in one launch, otherwise
// weight by weight.  Returns the weights after the last step and the loss of every step.
template <typename S>
int mlp_train(int rule, int together, float lr, float clip, int steps, int batch, int n_layers, const int* dims,
              const int* acts, const float* x, const int* labels, const float* const* W, const float* const* b,
              float* out_losses, float* const* out_W, float* const* out_b, float* out_update_ms) {
  auto X = data_from<S>({dims[0], batch}, x, false);
  auto Y = Data<Int>(cpu(), Shape{batch});
  for (int i = 0; i < batch; ++i) Y->value().v()[i] = labels[i];
  Y->move_to(gpu());
  Y->set_has_grad(false);
  std::vector<Ptr<WeightNode<S>>> Ws, bs, all;
  NodePtr<S> h = X;
  for (int l = 0; l < n_layers; ++l) {
    Ws.push_back(weight_from<S>({dims[l + 1], dims[l]}, W[l]));
    bs.push_back(weight_from<S>({dims[l + 1]}, b[l]));
    all.push_back(Ws[l]);
    all.push_back(bs[l]);
    h = make_ptr<AffineNode<S>>(make_op<S>(acts[l]), std::vector<NodePtr<S>>{Ws[l], h, bs[l]});
  }
  auto loss = Sum(PickNegLogSoftmax(h, Y));
  Graph g(loss);
  std::unique_ptr<Updater<S>> updater;
  if (rule == 0) updater = std::make_unique<update::Sgd<S>>(lr, clip);
  else updater = std::make_unique<update::Adam<S>>(lr, clip);
  double update_ms = 0;
  for (int step = 0; step < steps; ++step) {
    g.reset_forwarded();
    g.forward();
    g.reset_grad();
    g.backward(1.);
    read_back(loss->value(), out_losses ? out_losses + step : nullptr);
    gpu()->synchronize();
    const double t0 = now_ms();
    if (together) updater->update(g);
    else for (auto& w : all) updater->update(w);
    gpu()->synchronize();
    update_ms += now_ms() - t0;
  }
  if (out_update_ms) *out_update_ms = static_cast<float>(update_ms / std::max(1, steps));
  for (int l = 0; l < n_layers; ++l) {
    read_back(Ws[l]->value(), out_W[l]);
    read_back(bs[l]->value(), out_b[l]);
  }
  return 0;
}

// ---- the reference's Autobatch equivalence cases --------------------------------

struct Inputs {
  std::vector<Ptr<DataNode<Real>>> nodes;
  const float* const* vals;
  size_t next = 0;
  Ptr<DataNode<Real>> make(const Shape& s) {
    auto x = data_from<Real>(s, vals[next++], true);
    nodes.push_back(x);
    return x;
  }
};

// Builds case `which` over `in`; returns the scalar sink.
NodePtr<Real> autobatch_graph(int which, Inputs& in) {
  if (which == 0) {  // "Autobatch grad": two stacked Affines sharing operands
    auto x = in.make({2, 2}), y = in.make({2, 2}), b = in.make({2});
    auto h = Affine(x, y, x, y, b);
    auto t = Affine(h, y, b);
    return Sum(t);
  }
  // "Recurrent" (1) and "Recurrent mixed" (2): 3 sequences of 4 steps; 3 = "Recurrent" with tanh Affines
  std::vector<NodePtr<Real>> x;
  for (int i = 0; i < 12; ++i) x.push_back(in.make({2, 1}));
  auto W = in.make({3, 2}), V = in.make({3, 3}), b = in.make({3, 1});
  std::vector<NodePtr<Real>> hs;
  for (int i = 0; i < 3; ++i) {
    NodePtr<Real> h = Zero<Real>(gpu(), Shape{3, 1});
    for (int t = 0; t < 4; ++t) {
      if (which == 2 && (i + t) % 2 == 0)
        h = Add(W * x.at(4 * i + t), V * h, NodePtr<Real>(b));
      else if (which == 3)  // an Affine that carries a nonlinearity (not among the reference's cases)
        h = Affine<TanhOp>(W, x.at(4 * i + t), V, h, b);
      else
        h = Affine(W, x.at(4 * i + t), V, h, b);
    }
    hs.push_back(h);
  }
  return Sum(Add(hs));
}

// Whether Autobatch merges a group into one GatherProd (right operands read in
// place) instead of RowwiseCat + Prod.
bool g_autobatch_gather = false;

int count_prods(const Graph& g) {
  int n = 0;
  for (auto& node : g.nodes())
    if (dynamic_cast<ProdNode<Real>*>(node.get()) || dynamic_cast<GatherProdNode<Real>*>(node.get())) ++n;
  return n;
}

int autobatch_case(int which, const float* const* vals, float* sink_before, float* sink_after,
                   float* const* grads_before, float* const* grads_after, int* prods_before, int* prods_after) {
  Inputs in;
  in.vals = vals;
  auto s = autobatch_graph(which, in);
  Graph g(s);
  g.forward();
  g.reset_grad();
  g.backward(1.);
  read_back(s->value(), sink_before);
  for (size_t i = 0; i < in.nodes.size(); ++i) read_back(in.nodes[i]->grad(), grads_before[i]);
  *prods_before = count_prods(g);

  g = Autobatch(g, g_autobatch_gather);
  auto sink = dynamic_ptr_cast<Node<Real>>(g.sink());
  g.reset_forwarded();
  g.forward();
  g.reset_grad();
  g.backward(1.);
  read_back(sink->value(), sink_after);
  for (size_t i = 0; i < in.nodes.size(); ++i) read_back(in.nodes[i]->grad(), grads_after[i]);
  *prods_after = count_prods(g);
  return 0;
}

// ---- LSTM gates over ragged sequences ----------------------------------------------

int lstm(int mode, int nseq, const int* lens, int E, int H, const float* W, const float* b, const float* xs,
         const float* mask, int iters, float* out_h, float* out_loss, float* dW, float* db, float* dxs,
         float* out_ms, int* out_nodes, int* out_prods, int* out_launches, float* out_first_ms) {
  const bool autobatch = (mode & 1) != 0, level_exec = (mode & 2) != 0;
  Size total = 0;
  for (int s = 0; s < nseq; ++s) total += lens[s];
  auto Wn = weight_from<Real>({4 * H, E + H}, W);
  auto bn = weight_from<Real>({4 * H}, b);
  auto X = data_from<Real>({E, total}, xs, true);
  auto M = data_from<Real>({H, nseq}, mask, false);

  std::vector<NodePtr<Real>> finals;
  Size col = 0;
  for (int s = 0; s < nseq; ++s) {
    NodePtr<Real> h = Zero<Real>(place(), Shape{H, 1});
    NodePtr<Real> c = Zero<Real>(place(), Shape{H, 1});
    for (int t = 0; t < lens[s]; ++t, ++col) {
      auto x = Slice(NodePtr<Real>(X), Shape{0, col}, Shape{E, 1});
      auto z = Affine(Wn, Cat(NodePtr<Real>(x), h), bn);
      auto gate = [&](int k) { return Slice(NodePtr<Real>(z), Shape{k * H, 0}, Shape{H, 1}); };
      auto i = Sigmoid(gate(0));
      auto f = Sigmoid(gate(1));
      auto g = Tanh(gate(2));
      auto o = Sigmoid(gate(3));
      c = CwiseProd(f, c) + CwiseProd(i, g);
      h = CwiseProd(o, Tanh(c));
    }
    finals.push_back(h);
  }
  auto Hfin = RowwiseCat(finals);
  auto loss = Sum(CwiseProd(NodePtr<Real>(Hfin), NodePtr<Real>(M)));
  Graph g(loss);
  if (autobatch) {
    // The rewrite reads operand shapes (bias broadcast width), so the graph has
    // been evaluated once before it, as in test/autobatch.cpp:36-49.
    g.forward();
    g = Autobatch(g, g_autobatch_gather);
  }
  auto sink = dynamic_ptr_cast<Node<Real>>(g.sink());
  if (out_nodes) *out_nodes = static_cast<int>(g.nodes().size());
  if (out_prods) *out_prods = count_prods(g);
  double ms, first_ms;
  if (level_exec) {
    LevelExecutor ex(g);
    first_ms = run_passes(ex, 1);  // builds the launch plans and uploads their tables
    if (out_launches) *out_launches = static_cast<int>(ex.launches());  // table launches of one pass
    if (mode & 4) ex.freeze();     // the graph stays as it is: replay without re-describing
    if ((mode & 20) == 20) {       // ... with the launches of consecutive levels joined into chains
      ex.fuse();
      if (out_launches) {
        const size_t before = ex.launches();
        run_passes(ex, 1);
        *out_launches = static_cast<int>(ex.launches() - before);
      }
    }
    if ((mode & 12) == 12) {       // ... as one recorded device graph
      ex.record_pass();
      g_recorded_kernels = static_cast<long>(ex.recorded_kernels());
      ex.replay_pass();
      FillCount count;
      ms = run_replays(ex, iters);
    } else {
      FillCount count;
      ms = run_passes(ex, iters);
    }
  } else {
    first_ms = run_passes(g, 1);
    FillCount count;
    ms = run_passes(g, iters);
    if (out_launches) *out_launches = 0;
  }
  if (out_first_ms) *out_first_ms = static_cast<float>(first_ms);
  if (out_ms) *out_ms = static_cast<float>(ms);
  read_back(Hfin->value(), out_h);
  read_back(sink->value(), out_loss);
  read_back(Wn->grad(), dW);
  read_back(bn->grad(), db);
  read_back(X->grad(), dxs);
  return 0;
}

// ---- decoder layer of a GPT (examples/min-gpt.cu.cpp:93-163,227-235,293-301) -------------
//
// params, in order: ln1_g ln1_b Wk bk Wq bq Wv bv Wp bp ln2_g ln2_b W1 b1 W2 b2 lnf_g lnf_b Wh bh.
template <typename S>
int gpt_layer(int C, int nh, int B, int T, int V, const float* x, const int* targets, const float* const* params,
              int iters, float* out_loss, float* const* out_grads, float* out_dx, float* out_ms,
              int* out_nodes) {
  const Size hs = C / nh;
  const Shape shapes[20] = {{C}, {C}, {C, C}, {C}, {C, C}, {C}, {C, C}, {C}, {C, C}, {C},
                            {C}, {C}, {4 * C, C}, {4 * C}, {C, 4 * C}, {C}, {C}, {C}, {V, C}, {V}};
  std::vector<Ptr<WeightNode<S>>> w;
  for (int i = 0; i < 20; ++i) w.push_back(weight_from<S>(shapes[i], params[i]));
  enum { ln1_g, ln1_b, Wk, bk, Wq, bq, Wv, bv, Wp, bp, ln2_g, ln2_b, W1, b1, W2, b2, lnf_g, lnf_b, Wh, bh };

  auto X = data_from<S>({C, B, T}, x, true);
  auto Y = Data<Int>(cpu(), Shape{B * T});
  for (int i = 0; i < B * T; ++i) Y->value().v()[i] = targets[i];
  Y->move_to(place());
  Y->set_has_grad(false);

  auto ln = [&](const NodePtr<S>& v, int g, int b) -> NodePtr<S> {
    return CwiseProdAdd(NodePtr<S>(LayerNorm(v)), NodePtr<S>(w[g]), NodePtr<S>(w[b]), 1.f);
  };
  auto rearrange = [&](const NodePtr<S>& t, Shape perm) -> NodePtr<S> {
    return Permute(NodePtr<S>(Reshape(t, Shape{hs, nh, B, T})), std::move(perm));
  };

  // causal self-attention
  NodePtr<S> a1 = ln(X, ln1_g, ln1_b);
  auto k = rearrange(Affine(w[Wk], a1, w[bk]), {3, 0, 2, 1});  // T, hs, B, nh
  auto q = rearrange(Affine(w[Wq], a1, w[bq]), {0, 3, 2, 1});  // hs, T, B, nh
  auto v = rearrange(Affine(w[Wv], a1, w[bv]), {0, 3, 2, 1});  // hs, T, B, nh
  NodePtr<S> att = InPlaceProdScalar(NodePtr<S>(BatchedProd(k, q)), 1.f / std::sqrt(static_cast<float>(hs)));
  NodePtr<S> mask = Reshape(NodePtr<S>(UpperTri<S>(place(), static_cast<Size>(T))), Shape{T, T, 1, 1});
  att = InPlaceMask(att, mask, -std::numeric_limits<float>::infinity());
  att = Softmax(att);
  NodePtr<S> y = BatchedProd(v, att);  // hs, T, B, nh
  y = Permute(y, Shape{0, 3, 2, 1});   // hs, nh, B, T
  y = Affine(w[Wp], NodePtr<S>(Reshape(y, Shape{C, B, T})), w[bp]);
  NodePtr<S> y1 = NodePtr<S>(X) + y;

  // MLP
  NodePtr<S> a2 = ln(y1, ln2_g, ln2_b);
  auto h1 = Affine<GeluOp>(w[W1], NodePtr<S>(Reshape(a2, Shape{C, B * T})), w[b1]);
  auto h2 = Affine(w[W2], h1, w[b2]);
  NodePtr<S> y2 = y1 + NodePtr<S>(Reshape(NodePtr<S>(h2), Shape{C, B, T}));

  // final LayerNorm, vocabulary head, mean negative log-likelihood
  auto logits = Affine(w[Wh], ln(y2, lnf_g, lnf_b), w[bh]);
  auto loss = Mean(NodePtr<S>(PickNegLogSoftmax(NodePtr<S>(logits), Y)));

  Graph g(loss);
  if (out_nodes) *out_nodes = static_cast<int>(g.nodes().size());
  // With a training rule set, every pass ends with one update of all 20 weights (one launch).
  auto updater = make_updater<S>();
  std::vector<WeightPtr<S>> all(w.begin(), w.end());
  if (updater) g_after_backward = [&] { updater->update(all); };
  double ms;
  try {
    ms = run_warm(g, iters);
  } catch (...) {
    g_after_backward = nullptr;
    throw;
  }
  g_after_backward = nullptr;
  if (out_ms) *out_ms = static_cast<float>(ms);
  read_back(loss->value(), out_loss);
  for (int i = 0; i < 20; ++i) read_back(w[i]->grad(), out_grads[i]);
  read_back(X->grad(), out_dx);
  return 0;
}

#define GUARD(CALL)                    \
  try {                                \
    return CALL;                       \
  } catch (const std::exception& e) {  \
    g_error = e.what();                \
    return 2;                          \
  }

}  // namespace

extern "C" {

const char* scenario_last_error() { return g_error.c_str(); }

// Zero fills on demand during the timed passes of the last scenario (see g_timed_fills).
long scenario_timed_fills() { return g_timed_fills; }
// Kernel launches per pass (forward + reset_grad + backward) of the last scenario that was recorded
// as a device graph (executor mode with bit 3).
long scenario_recorded_kernels() { return g_recorded_kernels; }

// Columns summed so far by products that waited for the end of their backward pass
// (internal::LateOuterSum in ginn/node/prod.h).
long scenario_late_sum_columns() { return static_cast<long>(internal::late_outer_sum_columns().load()); }

// `steps` calls of one strided batched product, back to back on the context's
// stream and issued from native code, after `warmup` untimed ones: a product of
// a few microseconds can only be timed when the calls arrive faster than they
// run, which an interpreter's call overhead does not allow.  *out_ms = time per
// call between two events on that stream.
int scenario_time_batched_gemm(ginn_hip_ctx* ctx, int dtype, int op_a, int op_b, int m, int n, int k, const void* A,
                               int lda, long long stride_a, const void* B, int ldb, long long stride_b, float beta,
                               void* C, int ldc, long long stride_c, int batch, int warmup, int steps,
                               float* out_ms) {
  auto call = [&]() {
    return ginn_hip_gemm_strided_batched(ctx, static_cast<ginn_hip_dtype>(dtype), static_cast<ginn_hip_op>(op_a),
                                         static_cast<ginn_hip_op>(op_b), m, n, k, A, lda, stride_a, B, ldb, stride_b,
                                         beta, C, ldc, stride_c, batch);
  };
  int rc = 0;
  for (int i = 0; i < warmup && !rc; ++i) rc = call();
  if (!rc) rc = ginn_hip_event_record(ctx, 0);
  for (int i = 0; i < steps && !rc; ++i) rc = call();
  if (!rc) rc = ginn_hip_event_record(ctx, 1);
  if (!rc) rc = ginn_hip_sync(ctx);
  float ms = 0.f;
  if (!rc) rc = ginn_hip_event_elapsed_ms(ctx, 0, 1, &ms);
  if (rc) {
    g_error = ginn_hip_last_error();
    return rc;
  }
  *out_ms = ms / static_cast<float>(steps > 0 ? steps : 1);
  return 0;
}

int scenario_mlp(int dtype, int batch, int n_layers, const int* dims, const int* acts, const float* x,
                 const int* labels, const float* const* W, const float* const* b, int iters, float* out_loss,
                 float* out_nll, float* const* dW, float* const* db, float* out_ms) {
  switch (dtype) {
    case GINN_HIP_F32:
      GUARD(mlp<Real>(batch, n_layers, dims, acts, x, labels, W, b, iters, out_loss, out_nll, dW, db, out_ms));
    case GINN_HIP_F16:
      GUARD(mlp<Half>(batch, n_layers, dims, acts, x, labels, W, b, iters, out_loss, out_nll, dW, db, out_ms));
    case GINN_HIP_BF16:
      GUARD(mlp<BFloat16>(batch, n_layers, dims, acts, x, labels, W, b, iters, out_loss, out_nll, dW, db, out_ms));
  }
  g_error = "unknown dtype";
  return 1;
}

int scenario_mlp_train(int dtype, int rule, int together, float lr, float clip, int steps, int batch, int n_layers,
                       const int* dims, const int* acts, const float* x, const int* labels, const float* const* W,
                       const float* const* b, float* out_losses, float* const* out_W, float* const* out_b,
                       float* out_update_ms) {
  switch (dtype) {
    case GINN_HIP_F32:
      GUARD(mlp_train<Real>(rule, together, lr, clip, steps, batch, n_layers, dims, acts, x, labels, W, b,
                            out_losses, out_W, out_b, out_update_ms));
    case GINN_HIP_F16:
      GUARD(mlp_train<Half>(rule, together, lr, clip, steps, batch, n_layers, dims, acts, x, labels, W, b,
                            out_losses, out_W, out_b, out_update_ms));
    case GINN_HIP_BF16:
      GUARD(mlp_train<BFloat16>(rule, together, lr, clip, steps, batch, n_layers, dims, acts, x, labels, W, b,
                                out_losses, out_W, out_b, out_update_ms));
  }
  g_error = "unknown dtype";
  return 1;
}

int scenario_autobatch_case(int which, const float* const* vals, float* sink_before, float* sink_after,
                            float* const* grads_before, float* const* grads_after, int* prods_before,
                            int* prods_after) {
  GUARD(autobatch_case(which, vals, sink_before, sink_after, grads_before, grads_after, prods_before, prods_after));
}

// mode: bit 0 = rewrite the graph with Autobatch, bit 1 = run it through the level executor,
// bit 2 = freeze the executor after its first pass (the timed passes replay the recorded plans),
// bit 3 (with bit 2) = record the frozen pass as a device graph and time its replays,
// bit 4 (with bit 2) = join the table launches of consecutive levels into chain launches (out_launches
// then counts the table and chain launches of one such pass).
int scenario_lstm(int mode, int nseq, const int* lens, int E, int H, const float* W, const float* b,
                  const float* xs, const float* mask, int iters, float* out_h, float* out_loss, float* dW,
                  float* db, float* dxs, float* out_ms, int* out_nodes, int* out_prods, int* out_launches,
                  float* out_first_ms) {
  GUARD(lstm(mode, nseq, lens, E, H, W, b, xs, mask, iters, out_h, out_loss, dW, db, dxs, out_ms, out_nodes,
             out_prods, out_launches, out_first_ms));
}

// Executor of scenario_mlp and scenario_gpt_layer from now on: 0 = Graph (node by
// node), 2 = level executor, 6 = level executor frozen after its first pass, 14 = the frozen pass as a
// recorded device graph.
void scenario_set_executor(int mode) { g_exec_mode = mode; }
// 1: scenario_mlp, scenario_lstm (mode 0) and scenario_gpt_layer (executor 0) build and run their graphs on
// cpu() (the host layer's own loops, node by node); 0: on the HIP device.
void scenario_set_device(int on_cpu) { g_on_cpu = on_cpu != 0; }

// Training rule of scenario_gpt_layer from now on: -1 = none (forward + backward only), 0 = Sgd, 1 = Adam;
// every pass then ends with updater.update(all weights).  out_loss is the loss of the last pass.
void scenario_set_training(int rule, float lr, float clip) {
  g_train_rule = rule;
  g_train_lr = lr;
  g_train_clip = clip;
}

// Autobatch of scenario_autobatch_case and scenario_lstm from now on: 0 = the reference's rewrite
// (RowwiseCat + Prod + RowwiseUncat), 1 = one GatherProd per group.
void scenario_set_autobatch_gather(int gather) { g_autobatch_gather = gather != 0; }

int scenario_gpt_layer(int dtype, int C, int nh, int B, int T, int V, const float* x, const int* targets,
                       const float* const* params, int iters, float* out_loss, float* const* out_grads,
                       float* out_dx, float* out_ms, int* out_nodes) {
  switch (dtype) {
    case GINN_HIP_F32:
      GUARD(gpt_layer<Real>(C, nh, B, T, V, x, targets, params, iters, out_loss, out_grads, out_dx, out_ms, out_nodes));
    case GINN_HIP_F16:
      GUARD(gpt_layer<Half>(C, nh, B, T, V, x, targets, params, iters, out_loss, out_grads, out_dx, out_ms, out_nodes));
    case GINN_HIP_BF16:
      GUARD(gpt_layer<BFloat16>(C, nh, B, T, V, x, targets, params, iters, out_loss, out_grads, out_dx, out_ms,
                                out_nodes));
  }
  g_error = "unknown dtype";
  return 1;
}

}  // extern "C"
