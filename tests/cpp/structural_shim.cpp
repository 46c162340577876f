// Structural checks of the host layer, run on the HIP device: what the
// reference pins in test/tensor.cu.cpp (construction, copy, move, assignment
// across devices, resize, set, serialize, errors), test/graph.cpp:26-115
// (forwardedness, gradfulness, init_grad rules) and test/dev.cu.cpp:122-178
// (byte accounting of the preallocated device arena, tensors and nodes).
// The checks are written against the same public API a program written for the
// reference uses (Values<2>({{..}}), Tensor(dev, {shape}, {values}), x + y,
// Graph, PreallocGpu).  A failed check is recorded with its line and text;
// pytest calls shim_structural(case) and expects an empty report.
#include <sstream>
#include <string>
#include <vector>

#include <ginn/ginn.h>

using namespace ginn;
using namespace ginn::literals;

namespace {

thread_local std::string g_report;

#define CHECK(cond)                                                             \
  do {                                                                          \
    if (!(cond)) g_report += std::string("line ") + std::to_string(__LINE__) + ": " #cond "\n"; \
  } while (0)
#define CHECK_THROWS(stmt)                                                      \
  do {                                                                          \
    bool thrown__ = false;                                                      \
    try {                                                                       \
      stmt;                                                                     \
    } catch (const ginn::RuntimeError&) {                                       \
      thrown__ = true;                                                          \
    }                                                                           \
    if (!thrown__) g_report += std::string("line ") + std::to_string(__LINE__) + ": no RuntimeError from " #stmt "\n"; \
  } while (0)

template <typename Scalar>
std::vector<Scalar> one_to_six() {
  std::vector<Scalar> v;
  for (int i = 1; i <= 6; ++i) v.push_back(Scalar(i));
  return v;
}

template <typename Scalar>
Scalar sample_value() {
  if constexpr (std::is_same_v<Scalar, Int>) return 4;
  else return Scalar(0.6f);
}

template <typename Scalar>
bool all_equal(const Tensor<Scalar>& t, float val) {
  for (const Scalar& x : t.vector())
    if (!(static_cast<float>(x) == val)) return false;
  return true;
}

enum Maker { PLAIN, COPIED, MOVED, ASSIGNED_TO_GPU, ASSIGNED_TO_CPU };

// The five ways of obtaining a tensor from the same constructor arguments
// (test/tensor.cu.cpp:33-49), each checked for device, size, rank and values.
template <typename Scalar, typename... Args>
void made(Maker how, DeviceKind expect, Size size, size_t rank, const float* val, DevPtr init, Args... args) {
  using T = Tensor<Scalar>;
  auto check = [&](T& t) {
    CHECK(t.dev()->kind() == expect);
    CHECK(t.size() == size);
    if (rank) CHECK(t.shape().size() == rank);
    if (val) {
      t.move_to(cpu());
      for (Size i = 0; i < t.size(); ++i) CHECK(static_cast<float>(t.v()[i]) == *val);
    }
  };
  if (how == PLAIN) {
    T t(init, args...);
    check(t);
  } else if (how == COPIED) {
    T t_(init, args...);
    T t(t_);
    check(t);
  } else if (how == MOVED) {
    T t_(init, args...);
    T t(std::move(t_));
    check(t);
  } else {
    T t_(init, args...);
    T t(how == ASSIGNED_TO_GPU ? DevPtr(gpu()) : DevPtr(cpu()));
    t = t_;
    check(t);
  }
}

template <typename Scalar>
void tensor_ctors() {
  struct Row { Maker how; bool init_gpu; DeviceKind expect; };
  const Row rows[] = {{PLAIN, false, CPU}, {COPIED, false, CPU}, {MOVED, false, CPU}, {ASSIGNED_TO_CPU, false, CPU},
                      {PLAIN, true, GPU},  {COPIED, true, GPU},  {MOVED, true, GPU},  {ASSIGNED_TO_GPU, true, GPU},
                      {ASSIGNED_TO_CPU, true, CPU}};
  const Scalar val = sample_value<Scalar>();
  const float fval = static_cast<float>(val);
  for (const Row& r : rows) {
    const DevPtr init = r.init_gpu ? DevPtr(gpu()) : DevPtr(cpu());
    made<Scalar>(r.how, r.expect, 0, 0, nullptr, init);
    made<Scalar>(r.how, r.expect, 6, 3, nullptr, init, Shape{2, 1, 3});
    made<Scalar>(r.how, r.expect, 6, 3, &fval, init, Shape{2, 1, 3}, val);
  }
}

template <typename Scalar, typename DeviceType>
void tensor_resize_set_serialize_errors() {
  using T = Tensor<Scalar>;
  auto dev = std::make_shared<DeviceType>();
  auto fresh = [&] {
    T t(dev);
    t = T(dev, {2, 1, 3}, one_to_six<Scalar>());
    return t;
  };
  auto counts_up = [&](T& t) {
    t.move_to(cpu());
    for (Size i = 0; i < t.size(); ++i) CHECK(static_cast<float>(t.v()[i]) == static_cast<float>(i + 1));
  };
  {  // same size: contents stay
    T t = fresh();
    t.resize({6});
    CHECK(t.size() == 6);
    CHECK((t.shape() == Shape{6}));
    counts_up(t);
  }
  {
    T t = fresh();
    t.resize({2, 3});
    CHECK((t.shape() == Shape{2, 3}));
    counts_up(t);
  }
  {
    T t = fresh();
    t.resize({4});
    CHECK(t.size() == 4);
    CHECK((t.shape() == Shape{4}));
    t.resize({2, 2});
    CHECK((t.shape() == Shape{2, 2}));
  }
  {  // host access only on host tensors
    T t = fresh();
    if (dev->kind() == CPU) {
      CHECK(t.v() == t.data());
    } else {
      CHECK_THROWS(t.v());
    }
    // folds of the shape (views of rank 1..5 in the reference)
    CHECK((T::reduce(t.shape(), 1) == Shape{6}));
    CHECK((T::reduce(t.shape(), 2) == Shape{2, 3}));
    CHECK((T::reduce(t.shape(), 3) == Shape{2, 1, 3}));
    CHECK((T::reduce(t.shape(), 5) == Shape{2, 1, 3, 1, 1}));
    CHECK(t.rows() == 2 && t.cols() == 3);
  }
  {
    T t = fresh();
    t.set_zero();
    CHECK(all_equal(t, 0.f));
    t.set_ones();
    CHECK(all_equal(t, 1.f));
    Scalar val;
    if constexpr (std::is_same_v<Scalar, Int>) val = 12345;
    else val = Scalar(0.12345f);
    t.fill(val);
    CHECK(all_equal(t, static_cast<float>(val)));
  }
  if constexpr (std::is_same_v<Scalar, Real>) {
    T t = fresh();
    t.set_random();
    t.move_to(cpu());
    for (Size i = 0; i < t.size(); ++i) {
      CHECK(t.v()[i] <= 1.f && t.v()[i] >= -1.f);
      if (i > 0) CHECK(t.v()[i] != t.v()[i - 1]);
    }
  }
  {  // set(values...): as many as fit, the rest stays
    T t = fresh();
    t.set(5, 4, 3, 2, 1, 0);
    auto v = t.vector();
    for (size_t i = 0; i < v.size(); ++i) CHECK(static_cast<float>(v[i]) == 5.f - static_cast<float>(i));
    t.set(5, 4, 3, 2, 1, 0, 1, 2, 3);
    v = t.vector();
    for (size_t i = 0; i < v.size(); ++i) CHECK(static_cast<float>(v[i]) == 5.f - static_cast<float>(i));
    T u = fresh();
    u.set(5, 4, 3);
    v = u.vector();
    const float want[6] = {5, 4, 3, 4, 5, 6};
    for (size_t i = 0; i < 6; ++i) CHECK(static_cast<float>(v[i]) == want[i]);
  }
  {  // nested literal: element (i, j) is list[i][j]
    T t(dev);
    t.template set<2>(NestedInitList<2, Scalar>{{Scalar(1), Scalar(2), Scalar(3)}, {Scalar(4), Scalar(5), Scalar(6)}});
    CHECK((t.shape() == Shape{2, 3}));
    const auto v = t.vector();
    const float want[6] = {1, 4, 2, 5, 3, 6};  // column-major storage
    for (size_t i = 0; i < 6; ++i) CHECK(static_cast<float>(v[i]) == want[i]);
  }
  {
    T t = fresh(), t2(dev);
    std::ostringstream out;
    t.save(out);
    std::istringstream in(out.str());
    t2.load(in);
    CHECK(t == t2);
  }
  {
    T t1(dev, {1, 2}), t2(dev, {1, 3}), t3(dev);
    t3.map(t1, {2, 1});
    CHECK_THROWS(t3 = t2);
    CHECK_THROWS(t3.map(t2, {2, 1}));
    std::string msg;
    try {
      T bad(Shape{1, 3}, std::vector<Scalar>{Scalar(1), Scalar(2)});
    } catch (const ginn::RuntimeError& e) {
      msg = e.what();
    }
    CHECK(msg == "Size of Shape (3) does not match size of values (2)!");
  }
}

// test/graph.cpp:26-54, on the device (nodes compute there in this build).
void forwardedness() {
  auto make = [] {
    auto a = Identity(Data(gpu(), {2, 3}));
    auto b = Identity(Data(gpu(), {2, 3}));
    return std::make_pair(a, b);
  };
  {
    auto [a, b] = make();
    auto c = a + b;
    Graph g(c);
    CHECK(g.nodes().size() == 5);
    g.forward();
    for (const auto& e : g.nodes()) CHECK(e->forwarded);
  }
  {
    auto [a, b] = make();
    auto c = a + b;
    Graph(a).forward();
    CHECK(a->forwarded);
    CHECK(!b->forwarded);
    CHECK(!c->forwarded);
  }
  {
    auto [a, b] = make();
    auto c = a + b;
    Graph g(c);
    auto d = c + a;
    g.forward();
    for (const auto& e : g.nodes()) CHECK(e->forwarded);
    CHECK(!d->forwarded);
  }
}

// test/graph.cpp:56-113.
void gradfulness() {
  auto a = Random(gpu(), {2, 3});
  auto b = FixedRandom(gpu(), {2, 3});
  auto c = a + b;
  Graph g(c);
  CHECK(a->has_grad());
  CHECK(!b->has_grad());
  CHECK(c->has_grad());
  CHECK(a->grad().size() == 0);
  CHECK(b->grad().size() == 0);
  CHECK(c->grad().size() == 0);

  g.forward();
  g.init_grad();
  CHECK((a->grad().shape() == Shape{2, 3}));
  CHECK(b->grad().size() == 0);
  CHECK((c->grad().shape() == Shape{2, 3}));

  a->grad().fill(3.f);
  g.reset_grad();
  CHECK((a->grad().shape() == Shape{2, 3}));
  CHECK(all_equal(a->grad(), 0.f));
  CHECK(b->grad().size() == 0);
  CHECK(all_equal(c->grad(), 0.f));

  // init_grad keeps a gradient of the right size ...
  a->grad() = Tensor<Real>(gpu(), {2, 3}, {1, 2, 3, 4, 5, 6});
  g.init_grad();
  const auto kept = a->grad().vector();
  for (size_t i = 0; i < 6; ++i) CHECK(kept[i] == static_cast<float>(i + 1));
  // ... and replaces one of the wrong size
  a->grad() = Tensor<Real>(gpu(), {1, 3}, {1, 2, 3});
  g.init_grad();
  CHECK((a->grad().shape() == Shape{2, 3}));
}

// test/dev.cu.cpp:122-155: the arena counts exactly the bytes asked for.
template <typename Scalar>
void arena_tensors() {
  auto dev = PreallocGpu(100);
  Tensor<Scalar> t1(gpu(), {2, 3});
  CHECK(dev->used() == 0);
  Tensor<Scalar> t2(dev, {1, 2});
  CHECK(dev->used() == t2.size() * sizeof(Scalar));
  Tensor<Scalar> t3(dev);
  CHECK(dev->used() == t2.size() * sizeof(Scalar));
  t3 = t2;  // copies
  CHECK(dev->used() == 2 * t2.size() * sizeof(Scalar));
  auto t4 = t1.maybe_copy_to(dev);  // same GPU: a view, no copy
  CHECK(dev->used() == 2 * t2.size() * sizeof(Scalar));
  t1.move_to(dev);
  CHECK(dev->used() == (2 * t2.size() + t1.size()) * sizeof(Scalar));
  t2.move_to(dev);  // already there
  CHECK(dev->used() == (2 * t2.size() + t1.size()) * sizeof(Scalar));
  Tensor<Scalar> t5(cpu(), {1, 3});
  auto t6 = t5.maybe_copy_to(dev);  // from the host: a copy
  CHECK(dev->used() == (2 * t2.size() + t1.size() + t5.size()) * sizeof(Scalar));
  CHECK(dev->size() == 100);
  dev->clear();
  CHECK(dev->used() == 0);
}

// test/dev.cu.cpp:157-178, with the result of x + y checked as well: the
// operands sit back to back in the arena, 24 or 12 bytes apart.
template <typename Scalar>
void arena_nodes() {
  auto dev = PreallocGpu(200);
  auto x = Values<2>({{1, 2, 3}, {4, 5, 6}})->cast<Scalar>();
  auto y = Values<2>({{1, 2, 3}, {4, 5, 6}})->cast<Scalar>();
  x->set_has_grad(false);
  CHECK(dev->used() == 0);
  x->move_to(dev);
  CHECK(dev->used() == x->size() * sizeof(Scalar));
  y->move_to(dev);  // value and (empty) gradient
  CHECK(dev->used() == 2 * x->size() * sizeof(Scalar));
  auto z = x + y;
  Graph g(z);
  CHECK(dev->used() == 2 * x->size() * sizeof(Scalar));
  g.forward();
  CHECK(dev->used() == 3 * x->size() * sizeof(Scalar));
  g.reset_grad();  // z and y have gradients, x does not
  CHECK(dev->used() == 5 * x->size() * sizeof(Scalar));
  const auto v = z->value().vector();
  const float want[6] = {2, 8, 4, 10, 6, 12};
  for (size_t i = 0; i < 6; ++i) CHECK(static_cast<float>(v[i]) == want[i]);
  g.backward(1.);
  CHECK(all_equal(y->grad(), 1.f));
}

// A block that does not fit leaves the arena as it was; aligned arenas pad.
void arena_limits() {
  auto dev = PreallocGpu(100);
  Tensor<Real> a(dev, {24});  // 96 bytes: fits (96 < 100)
  CHECK(dev->used() == 96);
  CHECK_THROWS(Tensor<Real>(dev, {1}));  // 96 + 4 is not < 100
  CHECK(dev->used() == 96);
  auto al = PreallocGpuAligned(0, 1024, 256);
  Tensor<Half> h(al, {3});
  Tensor<Real> r(al, {2});
  CHECK(al->used() == 256 + 8);
  CHECK(reinterpret_cast<uintptr_t>(r.data()) % 256 == 0);
}

// The layout nodes on the HIP device with the known answers of test/nodes.cu.cpp:66-306 (Stack, Cat,
// RowwiseCat / RowwiseUncat, Reshape, RankView, Slice, Chip), for the floating scalars and for Int, which
// the reference instantiates them on as well.
template <typename Scalar>
Ptr<DataNode<Scalar>> on_gpu(const Ptr<DataNode<Real>>& x) {
  auto y = x->template cast<Scalar>();
  y->move_to(gpu());
  y->set_has_grad(false);
  return y;
}

template <typename Scalar, typename NodeT>
void expect_values(int line, const Ptr<NodeT>& node, const Shape& shape, const std::vector<float>& want) {
  Graph(node).forward();
  if (node->shape() != shape) g_report += "line " + std::to_string(line) + ": unexpected shape\n";
  const auto got = node->value().vector();
  if (got.size() != want.size()) {
    g_report += "line " + std::to_string(line) + ": unexpected size\n";
    return;
  }
  for (size_t i = 0; i < got.size(); ++i)
    if (static_cast<float>(got[i]) != want[i])
      g_report += "line " + std::to_string(line) + ": element " + std::to_string(i) + " differs\n";
}
#define EXPECT_VALUES(node, shape, ...) expect_values<Scalar>(__LINE__, node, shape, std::vector<float> __VA_ARGS__)

template <typename Scalar>
void layout_goldens() {
  using N = NodePtr<Scalar>;
  {  // Stack of rank-1 (test/nodes.cu.cpp:69-88): result[x, i, j] = nodes[i][j][x], column-major storage
    std::vector<N> v;
    for (int b = 0; b < 6; ++b) v.push_back(on_gpu<Scalar>(Values<1>({1.f + 4 * b, 2.f + 4 * b, 3.f + 4 * b, 4.f + 4 * b})));
    auto st = Stack<Scalar>({{v[0], v[1]}, {v[2], v[3]}, {v[4], v[5]}});
    // element (x, i, j) at x + 4 (i + 3 j) holds nodes[i][j][x] = 1 + x + 4 (2 i + j)
    std::vector<float> want(24);
    for (int j = 0; j < 2; ++j)
      for (int i = 0; i < 3; ++i)
        for (int x = 0; x < 4; ++x) want[x + 4 * (i + 3 * j)] = 1.f + x + 4 * (2 * i + j);
    expect_values<Scalar>(__LINE__, st, Shape{4, 3, 2}, want);
    CHECK(want[4 * (1 + 3 * 0) + 0] == 9.f);   // the literal's entry [0][1][0]
    CHECK(want[4 * (2 + 3 * 1) + 3] == 24.f);  // [3][2][1]
  }
  {  // Stack of rank-2 (:90-110)
    std::vector<N> v;
    for (int b = 0; b < 6; ++b)
      v.push_back(on_gpu<Scalar>(Values<2>({{1.f + 4 * b, 2.f + 4 * b}, {3.f + 4 * b, 4.f + 4 * b}})));
    auto st = Stack<Scalar>({{v[0], v[1]}, {v[2], v[3]}, {v[4], v[5]}});
    std::vector<float> want(24);
    for (int j = 0; j < 2; ++j)
      for (int i = 0; i < 3; ++i)
        for (int c = 0; c < 2; ++c)
          for (int r = 0; r < 2; ++r) want[r + 2 * c + 4 * (i + 3 * j)] = 1.f + (2 * r + c) + 4 * (2 * i + j);
    expect_values<Scalar>(__LINE__, st, Shape{2, 2, 3, 2}, want);
  }
  auto a12 = on_gpu<Scalar>(Values<2>({{1, 2}}));
  auto b22 = on_gpu<Scalar>(Values<2>({{3, 4}, {5, 6}}));
  auto c22 = on_gpu<Scalar>(Values<2>({{7, 8}, {9, 0}}));
  // Cat (:126-148): rows on top of each other; column-major: 1 3 5 7 9 | 2 4 6 8 0
  EXPECT_VALUES(Cat(N(a12), N(b22), N(c22)), (Shape{5, 2}), {1, 3, 5, 7, 9, 2, 4, 6, 8, 0});
  {  // RowwiseCat (:151-199)
    auto a = on_gpu<Scalar>(Values<2>({{1}, {2}}));
    auto b = on_gpu<Scalar>(Values<2>({{3, 4}, {5, 6}}));
    auto c = on_gpu<Scalar>(Values<2>({{7, 8, 9}, {0, 1, 2}}));
    auto cat = RowwiseCat(N(a), N(b), N(c));
    EXPECT_VALUES(cat, (Shape{2, 6}), {1, 2, 3, 5, 4, 6, 7, 0, 8, 1, 9, 2});
    CHECK((cat->offsets() == std::vector<Size>{0, 1, 3}));
    CHECK((cat->extents() == std::vector<Size>{1, 2, 3}));
    EXPECT_VALUES(RowwiseUncat(N(cat), 0, cat), (Shape{2, 1}), {1, 2});
    EXPECT_VALUES(RowwiseUncat(N(cat), 1, cat), (Shape{2, 2}), {3, 5, 4, 6});
    EXPECT_VALUES(RowwiseUncat(N(cat), 2, cat), (Shape{2, 3}), {7, 0, 8, 1, 9, 2});
  }
  {  // Reshape (:202-223) and RankView (:226-251): the same storage under other shapes
    auto W = on_gpu<Scalar>(Values<2>({{1, 2, 3, 4, 5, 6}}));
    EXPECT_VALUES(Reshape(N(W), Shape{6, 1}), (Shape{6, 1}), {1, 2, 3, 4, 5, 6});
    EXPECT_VALUES(Reshape(N(W), Shape{3, 2}), (Shape{3, 2}), {1, 2, 3, 4, 5, 6});
    EXPECT_VALUES(Reshape(N(W), Shape{3, 1, 2}), (Shape{3, 1, 2}), {1, 2, 3, 4, 5, 6});
    auto M = on_gpu<Scalar>(Values<2>({{1, 4}, {2, 5}, {3, 6}}));
    EXPECT_VALUES(RankView(N(M), 1), (Shape{6}), {1, 2, 3, 4, 5, 6});
    EXPECT_VALUES(RankView(N(M), 2), (Shape{3, 2}), {1, 2, 3, 4, 5, 6});
    EXPECT_VALUES(RankView(N(M), 3), (Shape{3, 2, 1}), {1, 2, 3, 4, 5, 6});
    CHECK_THROWS(RankView(N(M), 0));
  }
  {  // Slice (:254-286) and Chip (:288-306)
    auto x = on_gpu<Scalar>(Values<2>({{1, 2}, {3, 4}, {5, 6}, {7, 8}}));
    EXPECT_VALUES(Slice(N(x), Shape{1, 0}, Shape{3, 2}), (Shape{3, 2}), {3, 5, 7, 4, 6, 8});
    EXPECT_VALUES(Slice(N(x), Shape{0, 1}, Shape{4, 1}), (Shape{4, 1}), {2, 4, 6, 8});
    EXPECT_VALUES(Slice(N(x), Shape{2, 0}, Shape{2, 1}), (Shape{2, 1}), {5, 7});
    EXPECT_VALUES(Chip(N(x), 2, 0), (Shape{2}), {5, 6});
    EXPECT_VALUES(Chip(N(x), 1, 1), (Shape{4}), {2, 4, 6, 8});
  }
}

}  // namespace

// Arithmetic nodes with the known answers of test/nodes.cu.cpp:443-640 ("Add subtract": Add, AddScalar,
// Subtract, SubtractScalar, unary minus, ProdScalar, CwiseProd, CwiseProdAdd with and without a multiplier
// bias and broadcast operands, CwiseMax), forward, for the floating scalars and for Int.
template <typename Scalar>
void arithmetic_goldens() {
  using N = NodePtr<Scalar>;
  auto a = on_gpu<Scalar>(Values<2>({{1, 4}, {2, 5}, {3, 6}}));
  auto b = on_gpu<Scalar>(Values<2>({{-1, 4}, {-2, 5}, {-3, 6}}));
  auto c = on_gpu<Scalar>(Values<2>({{1, -4}, {2, -5}, {3, -6}}));
  const Shape s{3, 2};
  EXPECT_VALUES(Add(N(a), N(b)), s, {0, 0, 0, 8, 10, 12});
  EXPECT_VALUES(N(a) + N(b), s, {0, 0, 0, 8, 10, 12});
  EXPECT_VALUES(Add(N(a), N(b), N(c)), s, {1, 2, 3, 4, 5, 6});
  EXPECT_VALUES(N(a) + N(b) + N(c), s, {1, 2, 3, 4, 5, 6});
  EXPECT_VALUES(Add(N(a), N(b), N(a)), s, {1, 2, 3, 12, 15, 18});
  EXPECT_VALUES(AddScalar(a, 1), s, {2, 3, 4, 5, 6, 7});
  EXPECT_VALUES(a + 1, s, {2, 3, 4, 5, 6, 7});
  EXPECT_VALUES(1 + a, s, {2, 3, 4, 5, 6, 7});
  EXPECT_VALUES(Subtract(N(a), N(b)), s, {2, 4, 6, 0, 0, 0});
  EXPECT_VALUES(N(a) - N(b), s, {2, 4, 6, 0, 0, 0});
  EXPECT_VALUES(SubtractScalar(1, a), s, {0, -1, -2, -3, -4, -5});
  EXPECT_VALUES(1 - a, s, {0, -1, -2, -3, -4, -5});
  EXPECT_VALUES(1.0 - a, s, {0, -1, -2, -3, -4, -5});
  EXPECT_VALUES(AddScalar(a, -1), s, {0, 1, 2, 3, 4, 5});
  EXPECT_VALUES(a - 1, s, {0, 1, 2, 3, 4, 5});
  EXPECT_VALUES(-a, s, {-1, -2, -3, -4, -5, -6});
  EXPECT_VALUES(ProdScalar(a, 2), s, {2, 4, 6, 8, 10, 12});
  EXPECT_VALUES(a * 2, s, {2, 4, 6, 8, 10, 12});
  EXPECT_VALUES(2 * a, s, {2, 4, 6, 8, 10, 12});
  EXPECT_VALUES(CwiseProd(N(a), N(b)), s, {-1, -4, -9, 16, 25, 36});
  EXPECT_VALUES(CwiseProdAdd(N(a), N(b), N(c)), s, {0, -2, -6, 12, 20, 30});
  EXPECT_VALUES(CwiseProdAdd(N(a), N(b), N(c), Scalar(1)), s, {1, 0, -3, 16, 25, 36});  // a (b + 1) + c
  auto bv = on_gpu<Scalar>(Values<1>({-1, -2, -3}));
  auto cv = on_gpu<Scalar>(Values<1>({4, 5, 6}));
  EXPECT_VALUES(CwiseProdAdd(N(a), N(bv), N(cv)), s, {3, 1, -3, 0, -5, -12});
  EXPECT_VALUES(CwiseProdAdd(N(a), N(bv), N(cv), Scalar(1)), s, {4, 3, 0, 4, 0, -6});
  EXPECT_VALUES(CwiseMax(N(a), N(b), N(c)), s, {1, 2, 3, 4, 5, 6});
  EXPECT_VALUES(CwiseMax(N(b), N(c)), s, {1, 2, 3, 4, 5, 6});
}

// Select, Mask, Permute / Transpose / InPlacePermute, RowBroadcast / ColBroadcast and UpperTri with the known
// answers of test/nodes.cu.cpp:326-441, 825-880, forward, for the floating scalars and for Int (fractions are
// truncated by the cast to Int exactly as the reference's cast<Int>() truncates them).
template <typename Scalar>
void select_goldens() {
  using N = NodePtr<Scalar>;
  constexpr bool is_int = std::is_same_v<Scalar, Int>;
  // what a value turns into when it is stored as Scalar and read back
  auto q = [](float v) { return static_cast<float>(Scalar(v)); };
  auto qs = [&](std::vector<float> v) {
    for (auto& x : v) x = q(x);
    return v;
  };
  {  // Select (:825-858)
    auto if_ = Values<2>({{1., 0.}, {0., 1.}, {1., 0.}})->template cast<bool>();
    if_->move_to(gpu());
    if_->set_has_grad(false);
    auto a = on_gpu<Scalar>(Values<2>({{1., 2.}, {3., 4.}, {5., 6.}}));
    auto b = on_gpu<Scalar>(Values<2>({{.1, .2}, {.3, .4}, {.5, .6}}));
    const Shape s{3, 2};
    expect_values<Scalar>(__LINE__, Select(if_, N(a), N(b)), s, qs({1, .3f, 5, .2f, 4, .6f}));
    expect_values<Scalar>(__LINE__, Select(if_, N(a), Scalar(7)), s, {1, 7, 5, 7, 4, 7});
    expect_values<Scalar>(__LINE__, Select(if_, Scalar(7), N(b)), s, qs({7, .3f, 7, .2f, 7, .6f}));
    expect_values<Scalar>(__LINE__, Select(if_, Scalar(7), Scalar(-2)), s, {7, -2, 7, -2, 7, -2});
    if (is_int) CHECK(q(.3f) == 0.f);
  }
  {  // Mask (:860-885): a full mask and one that broadcasts over the columns
    auto mask = on_gpu<Scalar>(Values<2>({{1., 0.}, {0., 1.}, {1., 0.}}));
    auto mask2 = on_gpu<Scalar>(Values<2>({{1.}, {0.}, {1.}}));
    auto a = on_gpu<Scalar>(Values<2>({{1., 2.}, {3., 4.}, {5., 6.}}));
    EXPECT_VALUES(Mask(N(a), N(mask), Scalar(-1)), (Shape{3, 2}), {1, -1, 5, -1, 4, -1});
    EXPECT_VALUES(Mask(N(a), N(mask2), Scalar(7)), (Shape{3, 2}), {1, 7, 5, 2, 7, 6});
  }
  {  // Permute / Transpose / InPlacePermute (:326-380): a[i][j][k] = 1 + k + 4 j + 8 i, shape {3, 2, 4}
    const Shape dims{3, 2, 4};
    std::vector<float> av(24);
    for (int k = 0; k < 4; ++k)
      for (int j = 0; j < 2; ++j)
        for (int i = 0; i < 3; ++i) av[i + 3 * (j + 2 * k)] = 1.f + k + 4 * j + 8 * i;
    auto a0 = Values<3>({{{1, 2, 3, 4}, {5, 6, 7, 8}},
                         {{9, 10, 11, 12}, {13, 14, 15, 16}},
                         {{17, 18, 19, 20}, {21, 22, 23, 24}}});
    auto a = on_gpu<Scalar>(a0);
    expect_values<Scalar>(__LINE__, N(a) * 1, dims, av);  // the literal is laid out as the formula says
    // result[x] = a[y] with x[n] = y[perm[n]]
    auto permuted = [&](const Shape& perm, Shape& out_dims) {
      out_dims = {dims[perm[0]], dims[perm[1]], dims[perm[2]]};
      std::vector<float> w(24);
      Size y[3];
      for (y[2] = 0; y[2] < dims[2]; ++y[2])
        for (y[1] = 0; y[1] < dims[1]; ++y[1])
          for (y[0] = 0; y[0] < dims[0]; ++y[0]) {
            const Size x0 = y[perm[0]], x1 = y[perm[1]], x2 = y[perm[2]];
            w[x0 + out_dims[0] * (x1 + out_dims[1] * x2)] = av[y[0] + 3 * (y[1] + 2 * y[2])];
          }
      return w;
    };
    Shape od;
    {  // entries of the reference's literals b (perm 0 2 1), c (2 1 0) and e (1 2 0)
      auto w = permuted(Shape{0, 2, 1}, od);
      CHECK((od == Shape{3, 4, 2}));
      CHECK(w[0 + 3 * (1 + 4 * 0)] == 2.f && w[1 + 3 * (0 + 4 * 1)] == 13.f && w[2 + 3 * (3 + 4 * 1)] == 24.f);
      w = permuted(Shape{2, 1, 0}, od);
      CHECK((od == Shape{4, 2, 3}));
      CHECK(w[0 + 4 * (0 + 2 * 1)] == 9.f && w[1 + 4 * (1 + 2 * 2)] == 22.f && w[3 + 4 * (0 + 2 * 1)] == 12.f);
      w = permuted(Shape{1, 2, 0}, od);
      CHECK((od == Shape{2, 4, 3}));
      CHECK(w[0 + 2 * (1 + 4 * 1)] == 10.f && w[1 + 2 * (3 + 4 * 2)] == 24.f && w[1 + 2 * (0 + 4 * 1)] == 13.f);
    }
    for (const Shape& perm : {Shape{0, 2, 1}, Shape{2, 1, 0}, Shape{1, 0, 2}, Shape{1, 2, 0}, Shape{2, 0, 1},
                              Shape{0, 1, 2}}) {
      const auto w = permuted(perm, od);
      expect_values<Scalar>(__LINE__, Permute(N(a), perm), od, w);
      expect_values<Scalar>(__LINE__, InPlacePermute(N(a) * 1, perm), od, w);
    }
    expect_values<Scalar>(__LINE__, Transpose(N(a), 1, 2), Shape{3, 4, 2}, permuted(Shape{0, 2, 1}, od));
    expect_values<Scalar>(__LINE__, Transpose(N(a), 2, 0), Shape{4, 2, 3}, permuted(Shape{2, 1, 0}, od));
    expect_values<Scalar>(__LINE__, Transpose(N(a), 0, 1), Shape{2, 3, 4}, permuted(Shape{1, 0, 2}, od));
  }
  {  // RowBroadcast / ColBroadcast (:382-421)
    auto a = on_gpu<Scalar>(Values<2>({{1}, {2}, {3}}));
    auto b = on_gpu<Scalar>(Values<2>({{0.1, 1.2, 2.3}}));
    const auto b3 = qs({.1f, .1f, .1f, 1.2f, 1.2f, 1.2f, 2.3f, 2.3f, 2.3f});
    expect_values<Scalar>(__LINE__, RowBroadcast(N(b), 3), Shape{3, 3}, b3);
    expect_values<Scalar>(__LINE__, RowBroadcast(N(b), 1), Shape{1, 3}, qs({.1f, 1.2f, 2.3f}));
    expect_values<Scalar>(__LINE__, RowBroadcast(N(b), Dim(a, 0)), Shape{3, 3}, b3);
    expect_values<Scalar>(__LINE__, RowBroadcast(N(b), Dim(a, 1)), Shape{1, 3}, qs({.1f, 1.2f, 2.3f}));
    EXPECT_VALUES(ColBroadcast(N(a), 3), (Shape{3, 3}), {1, 2, 3, 1, 2, 3, 1, 2, 3});
    EXPECT_VALUES(ColBroadcast(N(a), 1), (Shape{3, 1}), {1, 2, 3});
    EXPECT_VALUES(ColBroadcast(N(a), Dim(b, 1)), (Shape{3, 3}), {1, 2, 3, 1, 2, 3, 1, 2, 3});
    EXPECT_VALUES(ColBroadcast(N(a), Dim(b, 0)), (Shape{3, 1}), {1, 2, 3});
  }
  {  // UpperTri (:423-441)
    EXPECT_VALUES(UpperTri<Scalar>(gpu(), 2), (Shape{2, 2}), {1, 0, 1, 1});
    std::vector<float> tri5(25);
    for (int c = 0; c < 5; ++c)
      for (int r = 0; r < 5; ++r) tri5[r + 5 * c] = r <= c ? 1.f : 0.f;
    expect_values<Scalar>(__LINE__, UpperTri<Scalar>(gpu(), 5), Shape{5, 5}, tri5);
  }
}

extern "C" {

// Runs the named group of checks; returns the report of failed checks ("" = all passed).
const char* shim_structural(const char* which) {
  g_report.clear();
  const std::string w(which);
  try {
    if (w == "tensor_ctors") {
      tensor_ctors<Real>();
      tensor_ctors<Int>();
      tensor_ctors<Half>();
      tensor_ctors<BFloat16>();
    } else if (w == "tensor_ops") {
      tensor_resize_set_serialize_errors<Real, GpuDevice>();
      tensor_resize_set_serialize_errors<Int, GpuDevice>();
      tensor_resize_set_serialize_errors<Half, GpuDevice>();
      tensor_resize_set_serialize_errors<BFloat16, GpuDevice>();
      tensor_resize_set_serialize_errors<Real, CpuDevice>();
      tensor_resize_set_serialize_errors<Int, CpuDevice>();
      tensor_resize_set_serialize_errors<Half, CpuDevice>();
    } else if (w == "forwardedness") {
      forwardedness();
    } else if (w == "gradfulness") {
      gradfulness();
    } else if (w == "arena_tensors") {
      arena_tensors<Real>();
      arena_tensors<Int>();
      arena_tensors<Half>();
    } else if (w == "arena_nodes") {
      arena_nodes<Real>();
      arena_nodes<Half>();
      arena_nodes<BFloat16>();
    } else if (w == "layout_goldens") {
      layout_goldens<Real>();
      layout_goldens<Half>();
      layout_goldens<BFloat16>();
      layout_goldens<Int>();
    } else if (w == "arithmetic_goldens") {
      arithmetic_goldens<Real>();
      arithmetic_goldens<Half>();
      arithmetic_goldens<BFloat16>();
      arithmetic_goldens<Int>();
    } else if (w == "select_goldens") {
      select_goldens<Real>();
      select_goldens<Half>();
      select_goldens<BFloat16>();
      select_goldens<Int>();
    } else if (w == "arena_limits") {
      arena_limits();
    } else {
      g_report = "unknown case " + w;
    }
  } catch (const std::exception& e) {
    g_report += std::string("exception: ") + e.what() + "\n";
  }
  return g_report.c_str();
}

}  // extern "C"
