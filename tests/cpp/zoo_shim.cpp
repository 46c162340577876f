// Test shim for the nodes around the product path (arithmetic, selection,
// picking, reductions, layout, in-place nodes): builds one node by name from
// host arrays on gpu(), runs the reference's protocol (test/check_node.h:27-121,
// test/testutil.h:93-171: e = f() + f(), loss = Sum(mask (*) e), forward,
// reset_grad, backward) and hands value and input gradients back as fp32.
// In-place nodes get `1 * x` as their first input, as the reference's tests do
// (test/nodes.cu.cpp:1202-1300), so that the two f() do not share storage.
#include <cmath>
#include <cstring>
#include <string>
#include <vector>

#include <ginn/ginn.h>

using namespace ginn;

namespace {

thread_local std::string g_zoo_error;

template <typename S>
Ptr<DataNode<S>> zoo_data(const Shape& shape, const float* vals, bool has_grad) {
  auto x = Data<S>(cpu(), shape);
  S* p = x->value().v();
  for (Size i = 0; i < x->value().size(); ++i) p[i] = S(vals[i]);
  x->move_to(gpu());
  x->set_has_grad(has_grad);
  return x;
}

template <typename T>
void zoo_read(const Tensor<T>& t, float* out) {
  if (!out) return;
  const auto v = t.vector();
  for (size_t i = 0; i < v.size(); ++i) out[i] = static_cast<float>(v[i]);
}

struct ZooArgs {
  const int* ip;
  const float* fp;
  const int* index;
  int n_index;
};

template <typename S>
DataPtr<Int> int_node(const Shape& shape, const int* vals) {
  auto x = Data<Int>(cpu(), shape);
  for (Size i = 0; i < x->value().size(); ++i) x->value().v()[i] = vals[i];
  x->move_to(gpu());
  x->set_has_grad(false);
  return x;
}

template <typename S>
NodePtr<bool> bool_node(const Shape& shape, const int* vals) {
  auto x = Data<bool>(cpu(), shape);
  for (Size i = 0; i < x->value().size(); ++i) x->value().v()[i] = vals[i] != 0;
  x->move_to(gpu());
  x->set_has_grad(false);
  return x;
}

// Builds the node `name` over the inputs; out_bool is set instead of the
// return value for bool-valued nodes.
template <typename S>
NodePtr<S> build(const std::string& name, const std::vector<Ptr<DataNode<S>>>& in, const ZooArgs& a,
                 NodePtr<bool>* out_bool) {
  auto X = [&](size_t i) { return NodePtr<S>(in.at(i)); };
  auto fresh = [&](size_t i) { return NodePtr<S>(1 * in.at(i)); };  // own storage per call
  const std::vector<Int> idx(a.index, a.index + a.n_index);
  if (name == "subtract") return Subtract(X(0), X(1));
  if (name == "subtract_op") return X(0) - X(1);
  if (name == "scalar_minus") return a.fp[0] - X(0);
  if (name == "minus_scalar") return X(0) - a.fp[0];
  if (name == "plus_scalar") return X(0) + a.fp[0];
  if (name == "scalar_plus") return a.fp[0] + X(0);
  if (name == "times_scalar") return X(0) * a.fp[0];
  if (name == "scalar_times") return a.fp[0] * X(0);
  if (name == "neg") return -X(0);
  if (name == "add3") return Add(X(0), X(1), X(2));
  if (name == "add_repeat") return X(0) + X(1) + X(0);
  if (name == "cwise_prod") return CwiseProd(X(0), X(1));
  if (name == "cwise_max") {
    std::vector<NodePtr<S>> all;
    for (size_t i = 0; i < in.size(); ++i) all.push_back(X(i));
    return CwiseMax(all);
  }
  if (name == "select_nn") return Select(bool_node<S>(in[0]->shape(), a.index), X(0), X(1));
  if (name == "select_ns") return Select(bool_node<S>(in[0]->shape(), a.index), X(0), S(a.fp[0]));
  if (name == "select_sn") return Select(bool_node<S>(in[0]->shape(), a.index), S(a.fp[0]), X(0));
  if (name == "select_ss") {
    Shape s(a.ip + 1, a.ip + 1 + a.ip[0]);
    return Select(bool_node<S>(s, a.index), S(a.fp[0]), S(a.fp[1]));
  }
  if (name == "mask") return Mask(X(0), X(1), a.fp[0]);
  if (name == "less_than") {
    *out_bool = X(0) < X(1);
    return nullptr;
  }
  if (name == "pick") return Pick(X(0), int_node<S>({static_cast<Size>(idx.size())}, a.index));
  if (name == "pick_vec") return Pick(X(0), idx);
  if (name == "pick_softmax") return PickSoftmax(X(0), idx);
  if (name == "pick_of_softmax") return Pick(Softmax(X(0)), idx);
  if (name == "pick_nls") return PickNegLogSoftmax(X(0), idx);
  if (name == "neg_log_pick_softmax") return -Log(PickSoftmax(X(0), idx));
  if (name == "pick_nlsig") return PickNegLogSigmoid(X(0), int_node<S>(in[0]->shape(), a.index));
  if (name == "chip") return Chip(X(0), a.ip[0], a.ip[1]);
  if (name == "axis_sum") return AxisSum(X(0), std::vector<Size>(a.ip + 1, a.ip + 1 + a.ip[0]));
  if (name == "variance") return Variance(X(0));
  if (name == "mean") return Mean(X(0));
  if (name == "sum") return Sum(X(0));
  if (name == "stack") {
    std::vector<std::vector<NodePtr<S>>> grid(static_cast<size_t>(a.ip[0]));
    for (int i = 0; i < a.ip[0]; ++i)
      for (int j = 0; j < a.ip[1]; ++j) grid[i].push_back(X(static_cast<size_t>(a.index[i * a.ip[1] + j])));
    return Stack<S>(grid);
  }
  if (name == "row_broadcast") return RowBroadcast(X(0), static_cast<Size>(a.ip[0]));
  if (name == "row_broadcast_dim") return RowBroadcast(X(0), Dim(BaseNodePtr(in.at(1)), a.ip[0]));
  if (name == "col_broadcast") return ColBroadcast(X(0), static_cast<Size>(a.ip[0]));
  if (name == "transpose") return Transpose(X(0), a.ip[0], a.ip[1]);
  if (name == "permute") return Permute(X(0), Shape(a.ip + 1, a.ip + 1 + a.ip[0]));
  if (name == "constant_like") return ConstantLike<S>(X(0), S(a.fp[0]));
  if (name == "ones_like") return OnesLike(in.at(0));
  if (name == "layernorm") return LayerNorm(X(0));
  if (name == "inplace_add") {
    std::vector<NodePtr<S>> all{fresh(0)};
    for (size_t i = 1; i < in.size(); ++i) all.push_back(X(i));
    return InPlaceAdd(all);
  }
  if (name == "inplace_add_repeat") return InPlaceAdd(fresh(0), X(1), X(1));
  if (name == "inplace_add_scalar") return InPlaceAddScalar(fresh(0), a.fp[0]);
  if (name == "inplace_cwise_prod") return InPlaceCwiseProd(fresh(0), X(1));
  if (name == "inplace_prod_scalar") return InPlaceProdScalar(fresh(0), a.fp[0]);
  if (name == "inplace_mask") return InPlaceMask(fresh(0), X(1), a.fp[0]);
  if (name == "inplace_sigmoid") return InPlaceSigmoid(fresh(0));
  if (name == "inplace_layernorm") return InPlaceLayerNorm(fresh(0));
  if (name == "inplace_permute") return InPlacePermute(fresh(0), Shape(a.ip + 1, a.ip + 1 + a.ip[0]));
  if (name == "inplace_dropout_p0") return InPlaceDropout(fresh(0), 0.);
  if (name == "dropout_p1") return Dropout(X(0), 1.);
  GINN_THROW("zoo: unknown node " + name);
  return nullptr;
}

template <typename S>
int zoo(const std::string& name, int n_in, const long* dims, const int* ranks, const float* const* vals,
        const int* has_grad, const ZooArgs& a, const float* mask, float* out_value, float* const* out_grads) {
  std::vector<Ptr<DataNode<S>>> in;
  const long* d = dims;
  for (int i = 0; i < n_in; ++i) {
    in.push_back(zoo_data<S>(Shape(d, d + ranks[i]), vals[i], has_grad[i] != 0));
    d += ranks[i];
  }
  if (!mask) {  // forward only
    NodePtr<bool> b;
    auto y = build<S>(name, in, a, &b);
    if (b) {
      Graph(b).forward();
      zoo_read(b->value(), out_value);
    } else {
      Graph(y).forward();
      zoo_read(y->value(), out_value);
    }
    gpu()->synchronize();
    return 0;
  }
  auto e = build<S>(name, in, a, nullptr) + build<S>(name, in, a, nullptr);
  Graph(e).forward();
  zoo_read(e->value(), out_value);
  auto m = zoo_data<S>(e->value().shape(), mask, false);
  auto loss = Sum(CwiseProd(NodePtr<S>(e), NodePtr<S>(m)));
  Graph g(loss);
  g.reset_forwarded();
  g.forward();
  g.reset_grad();
  g.backward(1.);
  gpu()->synchronize();
  for (int i = 0; i < n_in; ++i)
    if (has_grad[i] && out_grads[i]) zoo_read(in[static_cast<size_t>(i)]->grad(), out_grads[i]);
  return 0;
}

}  // namespace

#define ZOO_DISPATCH(dtype, CALL)                                              \
  try {                                                                        \
    switch (dtype) {                                                           \
      case GINN_HIP_F32: { using S = Real; return CALL; }                      \
      case GINN_HIP_F16: { using S = Half; return CALL; }                      \
      case GINN_HIP_BF16: { using S = BFloat16; return CALL; }                 \
    }                                                                          \
    g_zoo_error = "unknown dtype";                                             \
    return 1;                                                                  \
  } catch (const std::exception& e) {                                          \
    g_zoo_error = e.what();                                                    \
    return 2;                                                                  \
  }

extern "C" {

const char* zoo_last_error() { return g_zoo_error.c_str(); }

int shim_zoo(const char* name, int dtype, int n_in, const long* dims, const int* ranks, const float* const* vals,
             const int* has_grad, const int* ip, const float* fp, const int* index, int n_index, const float* mask,
             float* out_value, float* const* out_grads) {
  const ZooArgs a{ip, fp, index, n_index};
  ZOO_DISPATCH(dtype, zoo<S>(name, n_in, dims, ranks, vals, has_grad, a, mask, out_value, out_grads));
}

// Dropout on an all-ones tensor of n elements: value, and the input gradient
// for an all-ones output gradient (test/dropoutnodes.cu.cpp:30-106).  Two
// forward passes are run; `differs` reports whether their masks differ.
int shim_dropout(int dtype, int inplace, float p, long n, float* out_value, float* out_dx, int* differs) {
  ZOO_DISPATCH(dtype, ([&]() -> int {
    auto x = Data<S>(gpu(), Shape{n});
    x->value().fill(S(1.f));
    NodePtr<S> y;
    if (inplace) y = InPlaceDropout(1 * x, p);
    else y = Dropout(x, p);
    Graph g(y);
    g.forward();
    const auto first = y->value().vector();
    g.reset_forwarded();
    g.forward();
    zoo_read(y->value(), out_value);
    const auto second = y->value().vector();
    *differs = 0;
    for (size_t i = 0; i < first.size(); ++i)
      if (static_cast<float>(first[i]) != static_cast<float>(second[i])) *differs = 1;
    g.reset_grad();
    g.backward(1.);
    gpu()->synchronize();
    zoo_read(x->grad(), out_dx);
    return 0;
  })());
}

// argmax of a tensor along `dim` (flat when dim < 0), and the device-side
// uniform fill: n values in [-1, 1) from Tensor::set_random on a GPU tensor.
int shim_argmax(int dtype, const long* dims, int rank, const float* vals, int dim, long long* out) {
  ZOO_DISPATCH(dtype, ([&]() -> int {
    auto x = zoo_data<S>(Shape(dims, dims + rank), vals, false);
    if (dim < 0) {
      out[0] = static_cast<long long>(argmax(x->value()));
    } else {
      const auto v = argmax(x->value(), dim).vector();
      for (size_t i = 0; i < v.size(); ++i) out[i] = v[i];
    }
    return 0;
  })());
}

int shim_random(int dtype, long n, float* out_a, float* out_b) {
  ZOO_DISPATCH(dtype, ([&]() -> int {
    Tensor<S> a(gpu(), {n}), b(gpu(), {n});
    a.set_random();
    b.set_random();
    zoo_read(a, out_a);
    zoo_read(b, out_b);
    return 0;
  })());
}

// Construction-time and forward-time failures of these nodes (the CHECK_THROWS
// of test/nodes.cu.cpp:113-124, 976-977, test/dropoutnodes.cu.cpp:63-64):
// the message of the exception, "" if nothing was thrown.
const char* zoo_expect_throw(int which) {
  static thread_local std::string msg;
  msg.clear();
  try {
    auto a = Values<1>({1, 2, 3, 4}), b = Values<1>({5, 6, 7, 8}), e = Values<1>({17, 18, 19});
    for (auto* n : {&a, &b, &e}) (*n)->move_to(gpu());
    auto V = Random(gpu(), {2, 2, 3});
    switch (which) {
      case 0: Graph(Stack<Real>({{a, b}, {a, e}})).forward(); break;       // ragged input shapes
      case 1: Stack<Real>({{a, b}, {a}}); break;                           // ragged grid
      case 2: Stack<Real>({}); break;                                      // empty
      case 3: Stack<Real>({{}}); break;                                    // empty row
      case 4: AxisSum(V, {0, 0}); break;                                   // repeated axis
      case 5: AxisSum(V, {2, 0}); break;                                   // unsorted axes
      case 6: Dropout(V, -1.); break;
      case 7: Dropout(V, 1.1); break;
      case 8: Graph(Pick(V, std::vector<Int>{0, 1})).forward(); break;     // one index per column expected
      case 9: Graph(Chip(V, 2, 0)).forward(); break;                       // offset out of range
    }
  } catch (const std::exception& ex) {
    msg = ex.what();
  }
  return msg.c_str();
}

}  // extern "C"
