// Test shim: builds graphs with the header-only host layer (ginn_amd/ginn),
// runs them on gpu() and hands values and gradients back as fp32 host arrays.
// pytest drives it through ctypes and compares with the CPU oracle.  The
// protocol is the reference's (test/check_node.h:27-121, test/testutil.h:93-171):
// the checked expression is e = f() + f(), the loss is Sum(mask (*) e).
#include <algorithm>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include <ginn/ginn.h>

using namespace ginn;

namespace {

thread_local std::string g_error;
// Where the node cases below place their data: the HIP device, or cpu() for the host layer's own loops
// (shim_use_device).
bool g_on_cpu = false;

template <typename S>
Ptr<DataNode<S>> make_data(const Shape& shape, const float* vals, bool has_grad) {
  auto x = Data<S>(cpu(), shape);
  S* p = x->value().v();
  for (Size i = 0; i < x->value().size(); ++i) p[i] = S(vals[i]);
  if (!g_on_cpu) x->move_to(gpu());
  x->set_has_grad(has_grad);
  return x;
}

template <typename S>
void read_back(const Tensor<S>& t, float* out) {
  if (!out) return;
  const auto v = t.vector();
  for (size_t i = 0; i < v.size(); ++i) out[i] = static_cast<float>(v[i]);
}

Shape to_shape(const long* dims, int rank) { return Shape(dims, dims + rank); }

// loss = Sum(mask (*) (e + e)); forward, reset_grad, backward(1).
template <typename S>
void run_masked(const NodePtr<S>& e1, const NodePtr<S>& e2, const float* mask, float* out_value) {
  auto e = e1 + e2;
  Graph(e).forward();  // shapes are needed to size the mask
  read_back(e->value(), out_value);
  auto m = make_data<S>(e->value().shape(), mask, false);
  auto loss = Sum(CwiseProd(NodePtr<S>(e), NodePtr<S>(m)));
  Graph g(loss);
  g.reset_forwarded();
  g.forward();
  g.reset_grad();
  g.backward(1.);
  if (!g_on_cpu) gpu()->synchronize();
}

template <typename S>
int prod_node(int batched, const long* a_dims, int a_rank, const long* b_dims, int b_rank, const float* a,
              const float* b, const float* mask, float* out_value, float* out_da, float* out_db) {
  auto A = make_data<S>(to_shape(a_dims, a_rank), a, true);
  auto B = make_data<S>(to_shape(b_dims, b_rank), b, true);
  auto f = [&]() -> NodePtr<S> {
    if (batched) return BatchedProd(A, B);
    return Prod(A, B);
  };
  run_masked<S>(f(), f(), mask, out_value);
  read_back(A->grad(), out_da);
  read_back(B->grad(), out_db);
  return 0;
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
    case GINN_HIP_ACT_SOFTMAX: return std::make_unique<SoftmaxOp<S>>();
    case GINN_HIP_ACT_LOG: return std::make_unique<LogOp<S>>();
    case GINN_HIP_ACT_SQRT: return std::make_unique<SqrtOp<S>>();
  }
  GINN_THROW("unknown activation");
  return nullptr;
}

// ins: pairs * 2 + 1 tensors [A0, B0, ..., bias]; shapes given flat.
template <typename S>
int affine_node(int act, int n_ins, const long* dims, const int* ranks, const float* const* vals,
                const int* has_grad, const float* mask, float* out_value, float* const* out_grads) {
  std::vector<Ptr<DataNode<S>>> data;
  std::vector<NodePtr<S>> ins;
  const long* d = dims;
  for (int i = 0; i < n_ins; ++i) {
    data.push_back(make_data<S>(to_shape(d, ranks[i]), vals[i], has_grad[i] != 0));
    ins.push_back(data.back());
    d += ranks[i];
  }
  auto f = [&]() -> NodePtr<S> { return make_ptr<AffineNode<S>>(make_op<S>(act), ins); };
  run_masked<S>(f(), f(), mask, out_value);
  for (int i = 0; i < n_ins; ++i)
    if (has_grad[i]) read_back(data[i]->grad(), out_grads[i]);
  return 0;
}

template <typename S>
int nonlin_node(int act, const long* dims, int rank, const float* x, const float* mask, float* out_value,
                float* out_dx) {
  auto X = make_data<S>(to_shape(dims, rank), x, true);
  auto f = [&]() -> NodePtr<S> {
    switch (act) {
      case GINN_HIP_ACT_IDENTITY: return Identity(X);
      case GINN_HIP_ACT_TANH: return Tanh(X);
      case GINN_HIP_ACT_RELU: return Relu(X);
      case GINN_HIP_ACT_SIGMOID: return Sigmoid(X);
      case GINN_HIP_ACT_GELU: return Gelu(X);
      case GINN_HIP_ACT_GELU2: return Gelu2(X);
      case GINN_HIP_ACT_SOFTMAX: return Softmax(X);
      case GINN_HIP_ACT_LOG: return Log(X);
      case GINN_HIP_ACT_SQRT: return Sqrt(X);
    }
    GINN_THROW("unknown activation");
    return nullptr;
  };
  run_masked<S>(f(), f(), mask, out_value);
  read_back(X->grad(), out_dx);
  return 0;
}

#define DISPATCH(dtype, CALL)                                                  \
  try {                                                                        \
    switch (dtype) {                                                           \
      case GINN_HIP_F32: { using S = Real; return CALL; }                      \
      case GINN_HIP_F16: { using S = Half; return CALL; }                      \
      case GINN_HIP_BF16: { using S = BFloat16; return CALL; }                 \
    }                                                                          \
    g_error = "unknown dtype";                                                 \
    return 1;                                                                  \
  } catch (const std::exception& e) {                                          \
    g_error = e.what();                                                        \
    return 2;                                                                  \
  }

}  // namespace

extern "C" {

const char* shim_last_error() { return g_error.c_str(); }

int shim_gpus() { return gpus(); }

// 1: shim_prod_node, shim_affine_node, shim_nonlin_node and shim_mlp_on_cpu keep their graphs on cpu();
// 0 (the default): on the HIP device.
void shim_use_device(int on_cpu) { g_on_cpu = on_cpu != 0; }

int shim_prod_node(int dtype, int batched, const long* a_dims, int a_rank, const long* b_dims, int b_rank,
                   const float* a, const float* b, const float* mask, float* out_value, float* out_da,
                   float* out_db) {
  DISPATCH(dtype, prod_node<S>(batched, a_dims, a_rank, b_dims, b_rank, a, b, mask, out_value, out_da, out_db));
}

int shim_affine_node(int dtype, int act, int n_ins, const long* dims, const int* ranks, const float* const* vals,
                     const int* has_grad, const float* mask, float* out_value, float* const* out_grads) {
  DISPATCH(dtype, affine_node<S>(act, n_ins, dims, ranks, vals, has_grad, mask, out_value, out_grads));
}

int shim_nonlin_node(int dtype, int act, const long* dims, int rank, const float* x, const float* mask,
                     float* out_value, float* out_dx) {
  DISPATCH(dtype, nonlin_node<S>(act, dims, rank, x, mask, out_value, out_dx));
}

// The level executor against node-by-node execution on one graph whose input
// changes shape between passes: y = Tanh(x) (*) Sigmoid(x) + x + Relu(x) (x is
// used four times, so its gradient takes overlapping accumulations), loss =
// Sum(y (*) y).  Pass 1 runs `cols1` columns; then x is resized to `cols2`
// columns (the plans of the executor must notice and rebuild); with `frozen`
// the executor is frozen, replays once, is thawed, and only then sees the new
// shape.  Outputs: y and dx of the last pass from the executor and from
// Graph, and the number of plan (re)builds.
int shim_executor_replan(int rows, int cols1, int cols2, const float* x1, const float* x2, int frozen,
                         float* y_exec, float* dx_exec, float* y_plain, float* dx_plain, int* rebuilt) {
  try {
    auto x = make_data<Real>({rows, cols1}, x1, true);
    auto y = CwiseProd(Tanh(x), Sigmoid(x)) + x + Relu(x);
    auto loss = Sum(CwiseProd(NodePtr<Real>(y), NodePtr<Real>(y)));
    Graph g(loss);
    LevelExecutor ex(g);
    auto pass = [&](bool through_executor) {
      if (through_executor) {
        ex.reset_forwarded();
        ex.forward();
        ex.reset_grad();
        ex.backward(1.);
      } else {
        g.reset_forwarded();
        g.forward();
        g.reset_grad();
        g.backward(1.);
      }
      gpu()->synchronize();
    };
    pass(true);
    pass(true);  // same descriptions: the plans are reused
    const size_t built_once = ex.rebuilt();
    if (frozen) {
      ex.freeze();
      pass(true);
      if (ex.rebuilt() != built_once) throw std::runtime_error("a frozen pass rebuilt a plan");
      ex.thaw();
    }
    // new shape, new values
    auto fresh = make_data<Real>({rows, cols2}, x2, true);
    x->value() = fresh->value();
    pass(true);
    read_back(y->value(), y_exec);
    read_back(x->grad(), dx_exec);
    *rebuilt = static_cast<int>(ex.rebuilt() - built_once);
    pass(false);
    read_back(y->value(), y_plain);
    read_back(x->grad(), dx_plain);
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 1;
  }
}

// A recorded pass against the same pass run launch by launch: y = Tanh(W x + b)
// (*) x2 ..., loss = Sum(y (*) y) on a small MLP-like graph.  The executor is
// frozen and the pass recorded once; then, `replays` times, the input gets new
// values (an eager host-to-device copy between the replays), the recording is
// replayed, and values and gradients are compared with a launch-by-launch
// pass of the same frozen executor on the same input.  Returns the largest
// absolute difference seen (0 expected: the very same kernels and arguments).
int shim_executor_graph(int rows, int cols, int hidden, int replays, const float* w, const float* b,
                        const float* xs, float* max_diff) {
  try {
    auto W = make_data<Real>({hidden, rows}, w, true);
    auto B = make_data<Real>({hidden}, b, true);
    auto x = make_data<Real>({rows, cols}, xs, true);
    auto h = Affine<TanhOp>(W, x, B);
    auto y = CwiseProd(Sigmoid(h), h) + Relu(h);
    auto loss = Sum(CwiseProd(NodePtr<Real>(y), NodePtr<Real>(y)));
    Graph g(loss);
    LevelExecutor ex(g);
    auto pass = [&] {
      ex.reset_forwarded();
      ex.forward();
      ex.reset_grad();
      ex.backward(1.);
    };
    pass();
    ex.freeze();
    pass();
    ex.record_pass();
    float worst = 0.f;
    auto diff = [&](const std::vector<Real>& p, const std::vector<Real>& q) {
      for (size_t i = 0; i < p.size(); ++i) worst = std::max(worst, std::fabs(static_cast<float>(p[i] - q[i])));
    };
    for (int r = 0; r < replays; ++r) {
      auto fresh = make_data<Real>({rows, cols}, xs + static_cast<size_t>(r) * rows * cols, false);
      x->value() = fresh->value();  // same size: the storage stays, the values change
      ex.replay_pass();
      gpu()->synchronize();
      const auto y1 = y->value().vector(), dx1 = x->grad().vector(), dw1 = W->grad().vector(),
                 db1 = B->grad().vector();
      pass();
      gpu()->synchronize();
      diff(y1, y->value().vector());
      diff(dx1, x->grad().vector());
      diff(dw1, W->grad().vector());
      diff(db1, B->grad().vector());
    }
    *max_diff = worst;
    return 0;
  } catch (const std::exception& e) {
    g_error = e.what();
    return 1;
  }
}

// Two host threads drive the one context of gpu(0) at the same time
// (ginn/dev.h:203-212 hands every thread the same device object;
// examples/bench.cu.cpp:442-445 and mnist-dp.cu:158-172 do exactly this).
// Thread t computes C_t += A_t * B_t `iters` times through gpu_prod; the
// shapes are chosen by the caller so that the products keep partial sums in
// the context's workspace (split-K), which both threads share.  Outputs: C_0
// and C_1 after the last iteration (expected: iters * A_t * B_t).
int shim_two_threads(int dtype, int iters, const long* mnk0, const float* a0, const float* b0, float* c0,
                     const long* mnk1, const float* a1, const float* b1, float* c1) {
  DISPATCH(dtype, ([&]() -> int {
    const long* mnk[2] = {mnk0, mnk1};
    const float* as[2] = {a0, a1};
    const float* bs[2] = {b0, b1};
    float* cs[2] = {c0, c1};
    std::string errors[2];
    auto work = [&](int t) {
      try {
        auto A = make_data<S>({mnk[t][0], mnk[t][2]}, as[t], false);
        auto B = make_data<S>({mnk[t][2], mnk[t][1]}, bs[t], false);
        Tensor<S> C(gpu(), {mnk[t][0], mnk[t][1]});
        C.set_zero();
        for (int i = 0; i < iters; ++i)
          internal::gpu_prod(C, A->value(), B->value(), internal::ProdResult::Add);
        gpu()->synchronize();
        read_back(C, cs[t]);
      } catch (const std::exception& e) {
        errors[t] = e.what();
      }
    };
    std::thread other(work, 1);
    work(0);
    other.join();
    if (!errors[0].empty() || !errors[1].empty()) throw std::runtime_error(errors[0] + " " + errors[1]);
    return 0;
  })());
}

// Error paths of the host layer that need no kernel: returns the message of
// the exception thrown by `which`, or "" when nothing was thrown.
const char* shim_expect_throw(int which) {
  static thread_local std::string msg;
  msg.clear();
  try {
    switch (which) {
      case 0: {  // inner dimension mismatch in gpu_prod (ginn/prod.h:236)
        Tensor<Real> a(gpu(), {2, 3}), b(gpu(), {4, 2}), c(gpu(), {2, 2});
        internal::gpu_prod(c, a, b);
        break;
      }
      case 1: {  // BatchedProd on rank-2 inputs (ginn/node/prod.h:95-96)
        auto A = Data<Real>(gpu(), Shape{2, 3});
        auto B = Data<Real>(gpu(), Shape{3, 2});
        Graph(BatchedProd(A, B)).forward();
        break;
      }
      case 2: {  // Affine without a bias (ginn/node/affine.h:148-149)
        auto A = Data<Real>(gpu(), Shape{2, 3});
        auto B = Data<Real>(gpu(), Shape{3, 2});
        auto bad = make_ptr<AffineNode<Real>>(std::vector<NodePtr<Real>>{A, B});
        break;
      }
      case 3: {  // arena exhaustion (ginn/dev.h:238-241)
        auto dev = PreallocGpu(1024);
        Tensor<Real> t(dev, {1024});
        break;
      }
      case 4: {  // host access to a device tensor (ginn/tensor.h:328-329)
        Tensor<Real> t(gpu(), {4});
        t.v();
        break;
      }
      case 5: {  // a node without a host form refuses a cpu() tensor (the product-path nodes have one)
        auto A = Data<Real>(cpu(), Shape{2, 3});
        Graph(Variance(A)).forward();
        break;
      }
    }
  } catch (const std::exception& e) {
    msg = e.what();
  }
  return msg.c_str();
}

}  // extern "C"
