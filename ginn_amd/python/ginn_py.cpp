// Python module `ginn` over the host layer, with the call forms of the
// reference's ginn-py (ginn-py/ginn-py.cu.cpp:15-36 and the dev / tensor /
// node / init / update files beside it): devices; Real, Half, BFloat16, Int
// and Bool tensors exchanged with numpy; Data / Weight / Values / Random nodes
// with cast(scalar); Prod / BatchedProd / Affine, the nonlinearities and the
// arithmetic, layout, pick, select and reduce nodes for every floating scalar
// (the reference binds Real and Half, ginn-py/node/prod-py.cu.cpp:31-43,
// affine-py.cu.cpp:31-40; BFloat16 is this build's third one); operators on
// node handles; Graph, Autobatch, LevelExecutor; initialisers and updaters
// chosen by a `scalar` argument.  Nodes compute on the HIP device; numpy
// arrays enter and leave through host tensors.
#include <pybind11/numpy.h>
#include <pybind11/operators.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <sstream>

#include <ginn/autobatch.h>
#include <ginn/ginn.h>
#include <ginn/init/init.h>
#include <ginn/level_exec.h>
#include <ginn/update/update.h>

namespace py = pybind11;
using namespace ginn;

namespace {

template <typename T>
using SP = std::shared_ptr<T>;

enum class Scalar_ { Real, Half, BFloat16, Int, Bool };

template <typename S>
constexpr const char* prefix() {
  if constexpr (std::is_same_v<S, Real>) return "Real";
  else if constexpr (std::is_same_v<S, Half>) return "Half";
  else if constexpr (std::is_same_v<S, BFloat16>) return "BFloat16";
  else if constexpr (std::is_same_v<S, Int>) return "Int";
  else return "Bool";
}
template <typename S>
std::string named(const char* what) {
  return std::string(prefix<S>()) + what;
}

// What a tensor of S looks like in numpy: float32 for Real, float16 for Half
// (same bits), float32 for BFloat16 (numpy has no such type), int32, bool.
template <typename S>
struct np_of {
  using type = S;
};
template <>
struct np_of<BFloat16> {
  using type = float;
};
template <>
struct np_of<Half> {
  using type = uint16_t;  // carried as the raw bits of a float16 array
};

template <typename T>
SP<Node<typename T::Scalar>> as_node(const Ptr<T>& p) {
  return SP<Node<typename T::Scalar>>(p.as_shared_ptr());
}
template <typename S>
std::vector<NodePtr<S>> ptrs(const std::vector<SP<Node<S>>>& ins) {
  std::vector<NodePtr<S>> out;
  for (auto& n : ins) out.push_back(NodePtr<S>(n));
  return out;
}
template <typename S>
std::vector<WeightPtr<S>> wptrs(const std::vector<SP<WeightNode<S>>>& ws) {
  std::vector<WeightPtr<S>> out;
  for (auto& w : ws) out.push_back(WeightPtr<S>(w));
  return out;
}

// Column-major numpy array of a tensor's contents (copied through the host).
template <typename S>
py::array to_numpy(const Tensor<S>& t) {
  const std::vector<S> vals = t.vector();
  std::vector<py::ssize_t> shape(t.shape().begin(), t.shape().end());
  if constexpr (std::is_same_v<S, Half>) {
    std::vector<py::ssize_t> strides(shape.size());
    py::ssize_t step = 2;
    for (size_t d = 0; d < shape.size(); ++d) {
      strides[d] = step;
      step *= shape[d];
    }
    py::array a(py::dtype("float16"), shape, strides);
    auto* out = static_cast<uint16_t*>(a.mutable_data());
    for (size_t i = 0; i < vals.size(); ++i) out[i] = vals[i].bits;
    return a;
  } else {
    using N = typename np_of<S>::type;
    py::array_t<N, py::array::f_style> a(shape);
    N* out = a.mutable_data();
    for (size_t i = 0; i < vals.size(); ++i) out[i] = static_cast<N>(vals[i]);
    return std::move(a);
  }
}

// Any numeric array: converted to float32 (int32, bool) column-major by numpy, then to S.
template <typename S>
void from_numpy(Tensor<S>& t, const py::array& any) {
  using Host = std::conditional_t<is_floating_point_v<S>, float, S>;
  auto a = py::array_t<Host, py::array::f_style | py::array::forcecast>::ensure(any);
  if (!a) throw std::invalid_argument("cannot convert the array to the tensor's scalar type");
  Shape shape(a.shape(), a.shape() + a.ndim());
  if (shape.empty()) shape = {1};
  t.resize(shape);
  std::vector<S> vals(static_cast<size_t>(a.size()));
  for (size_t i = 0; i < vals.size(); ++i) vals[i] = S(a.data()[i]);
  t.set(vals);
}

template <typename S>
void bind_tensor(py::module_& m) {
  // values as Python hands them over (numbers or bools), converted to the tensor's scalar
  using Host = std::conditional_t<is_floating_point_v<S>, float, S>;
  auto with_values = [](const DevPtr& dev, const Shape& shape, const std::vector<Host>& val) {
    Tensor<S> t(dev, shape);
    std::vector<S> v(val.size());
    for (size_t i = 0; i < v.size(); ++i) v[i] = S(val[i]);
    t.set(v);
    return t;
  };
  // the constructors of ginn-py/tensor-py.cu.cpp:36-45
  py::class_<Tensor<S>>(m, named<S>("Tensor").c_str())
      .def(py::init([]() { return Tensor<S>(cpu(), Shape{0}); }))
      .def(py::init([](const DevPtr& dev) { return Tensor<S>(dev, Shape{0}); }), py::arg("device"))
      .def(py::init([](const Shape& shape) { return Tensor<S>(cpu(), shape); }), py::arg("shape"))
      .def(py::init([with_values](const Shape& shape, const std::vector<Host>& val) {
             return with_values(cpu(), shape, val);
           }),
           py::arg("shape"), py::arg("val"))
      .def(py::init([](const DevPtr& dev, const Shape& shape) { return Tensor<S>(dev, shape); }), py::arg("device"),
           py::arg("shape"))
      .def(py::init(with_values), py::arg("device"), py::arg("shape"), py::arg("val"))
      .def_property_readonly("dev", [](const Tensor<S>& t) { return t.dev(); })
      .def_property("shape", [](const Tensor<S>& t) { return t.shape(); },
                    [](Tensor<S>& t, const Shape& shape) { t.resize(shape); })
      .def_property_readonly("size", [](const Tensor<S>& t) { return t.size(); })
      .def_property_readonly("scalar", [](const Tensor<S>&) {
        if constexpr (std::is_same_v<S, Real>) return Scalar_::Real;
        else if constexpr (std::is_same_v<S, Half>) return Scalar_::Half;
        else if constexpr (std::is_same_v<S, BFloat16>) return Scalar_::BFloat16;
        else if constexpr (std::is_same_v<S, Int>) return Scalar_::Int;
        else return Scalar_::Bool;
      })
      .def("numpy", &to_numpy<S>)
      // m() / v(): the tensor as a matrix / vector.  Real and Int tensors on cpu() hand out a view of their own
      // memory that writes through, like the Eigen maps of ginn-py (ginn-py/test/test_tensor.py:114-127); the
      // other scalars and device tensors hand out a copy.
      .def("m", [](py::object self) -> py::object {
        Tensor<S>& t = self.cast<Tensor<S>&>();
        if constexpr (std::is_same_v<S, Real> || std::is_same_v<S, Int>) {
          if (t.dev()->kind() == CPU && t.size() > 0)
            return py::array_t<S>({static_cast<py::ssize_t>(t.rows()), static_cast<py::ssize_t>(t.cols())},
                                  {static_cast<py::ssize_t>(sizeof(S)), static_cast<py::ssize_t>(sizeof(S) * t.rows())},
                                  t.data(), self);
        }
        return to_numpy(t).attr("reshape")(py::make_tuple(t.rows(), t.cols()), py::arg("order") = "F");
      })
      .def("v", [](py::object self) -> py::object {
        Tensor<S>& t = self.cast<Tensor<S>&>();
        if constexpr (std::is_same_v<S, Real> || std::is_same_v<S, Int>) {
          if (t.dev()->kind() == CPU && t.size() > 0)
            return py::array_t<S>({static_cast<py::ssize_t>(t.size())}, {static_cast<py::ssize_t>(sizeof(S))}, t.data(),
                                  self);
        }
        return to_numpy(t).attr("reshape")(py::make_tuple(-1), py::arg("order") = "F");
      })
      .def("list", [](const Tensor<S>& t) {
        using Out = std::conditional_t<is_floating_point_v<S>, float, S>;
        std::vector<Out> out;
        for (const S& x : t.vector()) out.push_back(static_cast<Out>(x));
        return out;
      })
      // an array or nested lists: [[1, 2, 3], [4, 5, 6]] is a 2 x 3 tensor (ginn/tensor.h:331-395)
      .def("set", [](Tensor<S>& t, const py::object& values) {
        auto a = py::array::ensure(values);
        if (!a) throw std::invalid_argument("set() takes an array or nested lists of numbers");
        from_numpy<S>(t, a);
      })
      .def("item", [](const Tensor<S>& t) { return static_cast<std::conditional_t<is_floating_point_v<S>, float, S>>(t.item()); })
      .def("real", [](const Tensor<S>& t) { return t.template cast<Real>(); })
      .def("half", [](const Tensor<S>& t) { return t.template cast<Half>(); })
      .def("bfloat16", [](const Tensor<S>& t) { return t.template cast<BFloat16>(); })
      .def("int", [](const Tensor<S>& t) { return t.template cast<Int>(); })
      .def("bool", [](const Tensor<S>& t) { return t.template cast<bool>(); })
      .def("cast",
           [](const Tensor<S>& t, Scalar_ s) -> py::object {
             switch (s) {
               case Scalar_::Real: return py::cast(t.template cast<Real>());
               case Scalar_::Half: return py::cast(t.template cast<Half>());
               case Scalar_::BFloat16: return py::cast(t.template cast<BFloat16>());
               case Scalar_::Int: return py::cast(t.template cast<Int>());
               default: return py::cast(t.template cast<bool>());
             }
           })
      .def("set_ones", [](Tensor<S>& t) { t.set_ones(); })
      .def("set_zero", [](Tensor<S>& t) { t.set_zero(); })
      .def("set_random", [](Tensor<S>& t) { t.set_random(); })
      .def("fill", [](Tensor<S>& t, double v) { t.fill(S(static_cast<float>(v))); }, py::arg("val"))
      .def("move_to", [](Tensor<S>& t, const DevPtr& dev) { t.move_to(dev); }, py::arg("device"))
      .def("copy_to", [](const Tensor<S>& t, const DevPtr& dev) { return t.copy_to(dev); })
      .def("maybe_copy_to", [](Tensor<S>& t, const DevPtr& dev) { return t.maybe_copy_to(dev); })
      .def("__eq__", [](const Tensor<S>& a, const Tensor<S>& b) { return a == b; }, py::is_operator())
      .def("__repr__", [](const Tensor<S>& t) {
        std::ostringstream out;
        t.save(out);
        return out.str();
      })
      // the text form of Tensor::save / load
      .def("dumps", [](const Tensor<S>& t) {
        std::ostringstream out;
        t.save(out);
        return out.str();
      })
      .def("loads", [](Tensor<S>& t, const std::string& text) {
        std::istringstream in(text);
        t.load(in);
      });
}

template <typename S>
SP<DataNode<S>> cast_data(const DataNode<Real>& n) {
  return SP<DataNode<S>>(n.template cast<S>().as_shared_ptr());
}

template <typename S>
std::unique_ptr<NonlinOp<S>> nonlin_by_name(const std::string& n) {
  if (n == "identity") return std::make_unique<IdentityOp<S>>();
  if (n == "tanh") return std::make_unique<TanhOp<S>>();
  if (n == "relu") return std::make_unique<ReluOp<S>>();
  if (n == "sigmoid") return std::make_unique<SigmoidOp<S>>();
  if (n == "gelu") return std::make_unique<GeluOp<S>>();
  if (n == "gelu2") return std::make_unique<Gelu2Op<S>>();
  if (n == "softmax") return std::make_unique<SoftmaxOp<S>>();
  throw std::invalid_argument("unknown nonlinearity '" + n + "'");
}

// Node classes and the data / weight leaves of one scalar type.
template <typename S>
void bind_node_types(py::module_& m) {
  using N = Node<S>;
  auto node = py::class_<N, BaseNode, SP<N>>(m, named<S>("Node").c_str());
  node.def_property_readonly("value", [](N& n) -> Tensor<S>& { return n.value(); },
                             py::return_value_policy::reference_internal)
      .def_property_readonly("grad", [](N& n) -> Tensor<S>& { return n.grad(); },
                             py::return_value_policy::reference_internal)
      .def_property_readonly("shape", [](const N& n) { return n.shape(); })
      .def_property_readonly("size", [](const N& n) { return n.size(); })
      .def_property(
          "has_grad", [](const N& n) { return n.has_grad(); },
          [](N& n, bool hg) {
            if (auto* d = dynamic_cast<BaseDataNode<S>*>(&n)) d->set_has_grad(hg);
            else if (auto* w = dynamic_cast<WeightNode<S>*>(&n)) w->set_has_grad(hg);
            else throw std::invalid_argument("has_grad cannot be set on this node");
          });
  auto data = py::class_<DataNode<S>, N, SP<DataNode<S>>>(m, named<S>("DataNode").c_str());
  data.def("move_to", [](DataNode<S>& n, const DevPtr& dev) { n.move_to(dev); }, py::arg("device"))
      .def("set_random", [](DataNode<S>& n) { n.set_random(); })
      .def("fill", [](DataNode<S>& n, double v) { n.fill(S(static_cast<float>(v))); }, py::arg("val"));
  if constexpr (is_floating_point_v<S>) {
    py::class_<WeightNode<S>, N, SP<WeightNode<S>>>(m, named<S>("WeightNode").c_str())
        .def_property_readonly("id", &WeightNode<S>::id)
        .def("move_to", [](WeightNode<S>& n, const DevPtr& dev) { n.move_to(dev); }, py::arg("device"))
        .def("set_random", [](WeightNode<S>& n) { n.value().set_random(); })
        .def("reset_grad", [](WeightNode<S>& n) { n.reset_grad(); })
        .def("copy", [](WeightNode<S>& n, Copy mode) { return SP<WeightNode<S>>(n.copy(mode).as_shared_ptr()); },
             py::arg("mode"));
  }
}

// The nodes that exist for Int as well as for the floating scalars (ginn-py/node/common-py.cu.cpp:34-70,
// ginn-py/node/layout-py.cu.cpp, ginn-py/node/select-py.cu.cpp:33-46): arithmetic, layout, comparison, selection.
template <typename S>
void bind_shared_nodes(py::module_& m) {
  using N = Node<S>;
  using In = const SP<N>&;
  auto P = [](In x) { return NodePtr<S>(x); };
  m.def("Add", [](const std::vector<SP<N>>& ins) { return as_node(Add(ptrs<S>(ins))); });
  m.def("Add", [P](In a, In b) { return as_node(Add(P(a), P(b))); });
  m.def("Subtract", [P](In a, In b) { return as_node(Subtract(P(a), P(b))); });
  m.def("CwiseProd", [P](In a, In b) { return as_node(CwiseProd(P(a), P(b))); });
  m.def("CwiseMax", [](const std::vector<SP<N>>& ins) { return as_node(CwiseMax(ptrs<S>(ins))); });
  m.def("CwiseProdAdd",
        [P](In a, In b, In c, double bias) { return as_node(CwiseProdAdd(P(a), P(b), P(c), S(static_cast<float>(bias)))); },
        py::arg("in"), py::arg("multiplicand"), py::arg("addend"), py::arg("multiplicand_bias") = 0.);
  m.def("AddScalar", [P](In x, double s) { return as_node(AddScalar(P(x), s)); });
  m.def("SubtractScalar", [P](double s, In x) { return as_node(SubtractScalar(s, P(x))); });
  m.def("ProdScalar", [P](In x, double s) { return as_node(ProdScalar(P(x), s)); });
  m.def("Chip", [P](In x, Size offset, Size dim) { return as_node(Chip(P(x), offset, dim)); }, py::arg("in"),
        py::arg("offset"), py::arg("dim"));
  m.def("Reshape", [P](In x, const Shape& s) { return as_node(Reshape(P(x), s)); }, py::arg("in"), py::arg("shape"));
  m.def("RankView", [P](In x, Size rank) { return as_node(RankView(P(x), rank)); }, py::arg("in"), py::arg("rank"));
  m.def("Slice", [P](In x, const Shape& offsets, const Shape& sizes) { return as_node(Slice(P(x), offsets, sizes)); },
        py::arg("in"), py::arg("offsets"), py::arg("sizes"));
  m.def("Cat", [](const std::vector<SP<N>>& ins) { return as_node(Cat(ptrs<S>(ins))); });
  m.def("RowwiseCat", [](const std::vector<SP<N>>& ins) { return as_node(RowwiseCat(ptrs<S>(ins))); });
  m.def("Stack", [](const std::vector<std::vector<SP<N>>>& grid) {
    std::vector<std::vector<NodePtr<S>>> g;
    for (auto& row : grid) g.push_back(ptrs<S>(row));
    return as_node(Stack<S>(g));
  });
  m.def("LessThan", [P](In a, In b) { return SP<Node<bool>>(LessThan(P(a), P(b)).as_shared_ptr()); });
  m.def("Permute", [P](In x, const Shape& s) { return as_node(Permute(P(x), s)); }, py::arg("in"), py::arg("indices"));
  m.def("Transpose", [P](In x, Size i, Size j) { return as_node(Transpose(P(x), i, j)); }, py::arg("in"), py::arg("i"),
        py::arg("j"));
  m.def("RowBroadcast", [P](In x, Size rows) { return as_node(RowBroadcast(P(x), rows)); }, py::arg("in"), py::arg("size"));
  m.def("ColBroadcast", [P](In x, Size cols) { return as_node(ColBroadcast(P(x), cols)); }, py::arg("in"), py::arg("size"));
  m.def("RowBroadcast", [P](In x, const SP<DimNode>& rows) { return as_node(RowBroadcast(P(x), DimPtr(rows))); },
        py::arg("in"), py::arg("size"));
  m.def("ColBroadcast", [P](In x, const SP<DimNode>& cols) { return as_node(ColBroadcast(P(x), DimPtr(cols))); },
        py::arg("in"), py::arg("size"));
  m.def("Mask", [P](In x, In mask, double val) { return as_node(Mask(P(x), P(mask), val)); });
  m.def("Select", [P](const SP<Node<bool>>& c, In a, In b) { return as_node(Select(NodePtr<bool>(c), P(a), P(b))); });
  m.def("Select", [P](const SP<Node<bool>>& c, In a, double b) {
    return as_node(Select(NodePtr<bool>(c), P(a), S(static_cast<float>(b))));
  });
  m.def("Select", [P](const SP<Node<bool>>& c, double a, In b) {
    return as_node(Select(NodePtr<bool>(c), S(static_cast<float>(a)), P(b)));
  });
}

// Everything that computes, for one floating scalar type: overloads of the
// same Python name are told apart by the node type of their arguments.
template <typename S>
void bind_float_nodes(py::module_& m) {
  using N = Node<S>;
  using In = const SP<N>&;
  auto P = [](In x) { return NodePtr<S>(x); };

  m.def("Prod", [P](In a, In b) { return as_node(Prod(P(a), P(b))); });
  m.def("BatchedProd", [P](In a, In b) { return as_node(BatchedProd(P(a), P(b))); });
  m.def("Affine",
        [](const std::vector<SP<N>>& ins, const std::string& nonlin) {
          return as_node(make_ptr<AffineNode<S>>(nonlin_by_name<S>(nonlin), ptrs<S>(ins)));
        },
        py::arg("ins"), py::arg("nonlin") = "identity");
  bind_shared_nodes<S>(m);
  m.def("Dropout", [P](In x, double p) { return as_node(Dropout(P(x), static_cast<Real>(p))); });
#define GINN_PY_UNARY(F) m.def(#F, [P](In x) { return as_node(F(P(x))); })
  GINN_PY_UNARY(Identity);
  GINN_PY_UNARY(Sigmoid);
  GINN_PY_UNARY(Tanh);
  GINN_PY_UNARY(Relu);
  GINN_PY_UNARY(Gelu);
  GINN_PY_UNARY(Gelu2);
  GINN_PY_UNARY(Softmax);
  GINN_PY_UNARY(Log);
  GINN_PY_UNARY(Sqrt);
  GINN_PY_UNARY(Sum);
  GINN_PY_UNARY(Mean);
  GINN_PY_UNARY(Variance);
  GINN_PY_UNARY(LayerNorm);
#undef GINN_PY_UNARY
  m.def("AxisSum", [P](In x, const std::vector<Size>& axes) { return as_node(AxisSum(P(x), axes)); });
  auto index_of = [](const SP<DataNode<Int>>& i) { return DataPtr<Int>(i); };
  m.def("Pick", [P, index_of](In x, const SP<DataNode<Int>>& i) { return as_node(Pick(P(x), index_of(i))); });
  m.def("Pick", [P](In x, const std::vector<Int>& i) { return as_node(Pick(P(x), i)); });
  m.def("PickSoftmax", [P, index_of](In x, const SP<DataNode<Int>>& i) { return as_node(PickSoftmax(P(x), index_of(i))); });
  m.def("PickSoftmax", [P](In x, const std::vector<Int>& i) { return as_node(PickSoftmax(P(x), i)); });
  m.def("PickNegLogSoftmax",
        [P, index_of](In x, const SP<DataNode<Int>>& i) { return as_node(PickNegLogSoftmax(P(x), index_of(i))); });
  m.def("PickNegLogSoftmax", [P](In x, const std::vector<Int>& i) { return as_node(PickNegLogSoftmax(P(x), i)); });
  m.def("PickNegLogSigmoid",
        [P, index_of](In x, const SP<DataNode<Int>>& i) { return as_node(PickNegLogSigmoid(P(x), index_of(i))); });

  // initialisers and updaters of this scalar (chosen through `scalar=` below)
  py::class_<init::Xavier<S>>(m, named<S>("Xavier").c_str())
      .def("init", [](const init::Xavier<S>& i, const std::vector<SP<WeightNode<S>>>& ws) {
        for (auto& w : wptrs<S>(ws)) i.init(w);
      })
      .def("init", [](const init::Xavier<S>& i, const SP<WeightNode<S>>& w) { i.init(WeightPtr<S>(w)); });
  py::class_<init::Uniform<S>>(m, named<S>("Uniform").c_str())
      .def("init", [](const init::Uniform<S>& i, const std::vector<SP<WeightNode<S>>>& ws) {
        for (auto& w : wptrs<S>(ws)) i.init(w);
      })
      .def("init", [](const init::Uniform<S>& i, const SP<WeightNode<S>>& w) { i.init(WeightPtr<S>(w)); });
  py::class_<update::Sgd<S>>(m, named<S>("Sgd").c_str())
      .def_readwrite("lr", &update::Sgd<S>::lr)
      .def_readwrite("clip", &update::Sgd<S>::clip)
      .def("update", [](update::Sgd<S>& u, const std::vector<SP<WeightNode<S>>>& ws) { u.update(wptrs<S>(ws)); })
      .def("update", [](update::Sgd<S>& u, const SP<WeightNode<S>>& w) { u.update(WeightPtr<S>(w)); })
      .def("update", [](update::Sgd<S>& u, Graph& g) { u.update(g); });
  py::class_<update::Adam<S>>(m, named<S>("Adam").c_str())
      .def_readwrite("lr", &update::Adam<S>::lr_)
      .def_readwrite("clip", &update::Adam<S>::clip_)
      .def("update", [](update::Adam<S>& u, const std::vector<SP<WeightNode<S>>>& ws) { u.update(wptrs<S>(ws)); })
      .def("update", [](update::Adam<S>& u, const SP<WeightNode<S>>& w) { u.update(WeightPtr<S>(w)); })
      .def("update", [](update::Adam<S>& u, Graph& g) { u.update(g); });
}

// Operators on node handles (ginn-py/node/common-py.cu.cpp): x + y, x - y,
// x * y (the matrix product, as in the reference), x * 2, 2 * x, -x, x < y.
template <typename S>
void bind_operators(py::class_<Node<S>, BaseNode, SP<Node<S>>>& c) {
  using N = Node<S>;
  using In = const SP<N>&;
  auto P = [](In x) { return NodePtr<S>(x); };
  c.def("__add__", [P](In a, In b) { return as_node(Add(P(a), P(b))); })
      .def("__add__", [P](In a, double s) { return as_node(AddScalar(P(a), s)); })
      .def("__radd__", [P](In a, double s) { return as_node(AddScalar(P(a), s)); })
      .def("__sub__", [P](In a, In b) { return as_node(Subtract(P(a), P(b))); })
      .def("__sub__", [P](In a, double s) { return as_node(AddScalar(P(a), -s)); })
      .def("__rsub__", [P](In a, double s) { return as_node(SubtractScalar(s, P(a))); })
      .def("__mul__", [P](In a, double s) { return as_node(ProdScalar(P(a), s)); })
      .def("__rmul__", [P](In a, double s) { return as_node(ProdScalar(P(a), s)); })
      .def("__neg__", [P](In a) { return as_node(ProdScalar(P(a), -1.)); })
      .def("__lt__", [P](In a, In b) { return SP<Node<bool>>(LessThan(P(a), P(b)).as_shared_ptr()); });
  if constexpr (is_floating_point_v<S>) c.def("__mul__", [P](In a, In b) { return as_node(Prod(P(a), P(b))); });
}

// f<S>(args...) for the floating scalar named by `s`, as a Python object.
template <template <typename> class F, typename... Args>
py::object make_for(Scalar_ s, Args... args) {
  switch (s) {
    // (updaters hold mutexes: handed over by pointer, not by value)
    case Scalar_::Real: return py::cast(std::make_unique<F<Real>>(args...));
    case Scalar_::Half: return py::cast(std::make_unique<F<Half>>(args...));
    case Scalar_::BFloat16: return py::cast(std::make_unique<F<BFloat16>>(args...));
    default: throw std::invalid_argument("a floating-point scalar (Real, Half, BFloat16) is needed here");
  }
}

py::object data_node(const DevPtr& dev, const Shape& shape, Scalar_ s) {
  switch (s) {
    case Scalar_::Real: return py::cast(SP<DataNode<Real>>(Data<Real>(dev, shape).as_shared_ptr()));
    case Scalar_::Half: return py::cast(SP<DataNode<Half>>(Data<Half>(dev, shape).as_shared_ptr()));
    case Scalar_::BFloat16: return py::cast(SP<DataNode<BFloat16>>(Data<BFloat16>(dev, shape).as_shared_ptr()));
    case Scalar_::Int: return py::cast(SP<DataNode<Int>>(Data<Int>(dev, shape).as_shared_ptr()));
    default: return py::cast(SP<DataNode<bool>>(Data<bool>(dev, shape).as_shared_ptr()));
  }
}

}  // namespace

PYBIND11_MODULE(ginn, m) {
  m.doc() = "GINN graphs on the MI355X product path";
  py::register_exception<RuntimeError>(m, "RuntimeError", PyExc_RuntimeError);

  // ---- scalars (ginn-py/tensor-py.h:36-48): ginn.Real, ginn.Half, ginn.Int, ginn.Bool ----
  py::enum_<Scalar_>(m, "Scalar")
      .value("Real", Scalar_::Real)
      .value("Half", Scalar_::Half)
      .value("BFloat16", Scalar_::BFloat16)
      .value("Int", Scalar_::Int)
      .value("Bool", Scalar_::Bool)
      .export_values();
  py::enum_<Copy>(m, "Copy").value("Tied", Copy::Tied).value("Deep", Copy::Deep);

  // ---- devices (ginn-py/dev-py.cu.cpp) ----
  py::enum_<DeviceKind>(m, "DeviceKind").value("CPU", CPU).value("GPU", GPU).value("NULL_DEV", NULL_DEV);
  m.attr("DeviceType") = m.attr("DeviceKind");  // the reference's name of the enumeration
  py::class_<DeviceId>(m, "DeviceId")
      .def_readonly("kind", &DeviceId::kind)
      .def_readonly("idx", &DeviceId::idx)
      .def("__repr__",
           [](const DeviceId& i) {
             return std::string("<DeviceId with kind: ") + (i.kind == CPU ? "CPU" : i.kind == GPU ? "GPU" : "NULL_DEV") +
                    ", idx: " + std::to_string(i.idx) + ">";
           })
      .def("__eq__", [](const DeviceId& a, const DeviceId& b) { return a == b; }, py::is_operator());
  // Devices compare by identity, as in ginn-py (no __eq__ there): cpu() and gpu(i) hand out one object each,
  // Cpu() / Gpu(i) / the arenas a new one per call; ids compare by value.
  py::class_<Device, SP<Device>>(m, "Device")
      .def_property_readonly("kind", &Device::kind)
      .def_property_readonly("id", &Device::id)
      .def_property_readonly("idx", [](const Device& d) { return d.id().idx; })
      .def_property_readonly("precedence", &Device::precedence);
  py::class_<PreallocCpuDevice, Device, SP<PreallocCpuDevice>>(m, "PreallocCpuDevice")
      .def("clear", &PreallocCpuDevice::clear)
      .def_property_readonly("used", &PreallocCpuDevice::used)
      .def_property_readonly("size", &PreallocCpuDevice::size);
  py::class_<PreallocGpuDevice, Device, SP<PreallocGpuDevice>>(m, "PreallocGpuDevice")
      .def("clear", &PreallocGpuDevice::clear)
      .def_property_readonly("used", &PreallocGpuDevice::used)
      .def_property_readonly("size", &PreallocGpuDevice::size);
  m.def("cpu", []() -> SP<Device> { return cpu(); });
  m.def("Cpu", []() -> SP<Device> { return Cpu(); });
  m.def("gpu", [](int idx) -> SP<Device> { return gpu(idx); }, py::arg("gpu_idx") = 0);
  m.def("Gpu", [](size_t idx) -> SP<Device> { return Gpu(idx); }, py::arg("gpu_idx") = 0);
  m.def("gpus", &gpus);
  m.def("PreallocCpu", [](size_t bytes) { return PreallocCpu(bytes); }, py::arg("size"));
  m.def("PreallocGpu", [](size_t bytes) { return PreallocGpu(bytes); }, py::arg("size"));
  m.def("PreallocGpu", [](size_t idx, size_t bytes) { return PreallocGpu(idx, bytes); }, py::arg("idx"),
        py::arg("size"));

  // ---- tensors (ginn-py/tensor-py.cu.cpp) ----
  bind_tensor<Real>(m);
  bind_tensor<Half>(m);
  bind_tensor<BFloat16>(m);
  bind_tensor<Int>(m);
  bind_tensor<bool>(m);
  // Tensor(device, shape, scalar): the tensor class by scalar (ginn-py/tensor-py.cu.cpp:120-135)
  auto tensor_of = [](const DevPtr& dev, const Shape& shape, Scalar_ s) -> py::object {
    switch (s) {
      case Scalar_::Real: return py::cast(Tensor<Real>(dev, shape));
      case Scalar_::Half: return py::cast(Tensor<Half>(dev, shape));
      case Scalar_::BFloat16: return py::cast(Tensor<BFloat16>(dev, shape));
      case Scalar_::Int: return py::cast(Tensor<Int>(dev, shape));
      default: return py::cast(Tensor<bool>(dev, shape));
    }
  };
  m.def("Tensor", [tensor_of](Scalar_ s) { return tensor_of(cpu(), Shape{0}, s); }, py::arg("scalar") = Scalar_::Real);
  m.def("Tensor", [tensor_of](const DevPtr& dev, Scalar_ s) { return tensor_of(dev, Shape{0}, s); }, py::arg("device"),
        py::arg("scalar") = Scalar_::Real);
  m.def("Tensor", tensor_of, py::arg("device"), py::arg("shape"), py::arg("scalar") = Scalar_::Real);
  m.def("Tensor", [tensor_of](const Shape& shape, Scalar_ s) { return tensor_of(cpu(), shape, s); }, py::arg("shape"),
        py::arg("scalar") = Scalar_::Real);

  // ---- nodes (ginn-py/node-py.cu.cpp) ----
  py::class_<BaseNode, SP<BaseNode>>(m, "BaseNode")
      .def("forward", &BaseNode::forward)
      .def("reset_forwarded", &BaseNode::reset_forwarded)
      .def_readonly("forwarded", &BaseNode::forwarded)
      .def_property_readonly("name", &BaseNode::name)
      .def_property_readonly("dev", [](const BaseNode& n) { return n.dev(); });
  bind_node_types<Real>(m);
  bind_node_types<Half>(m);
  bind_node_types<BFloat16>(m);
  bind_node_types<Int>(m);
  bind_node_types<bool>(m);
  {
    auto real = py::class_<Node<Real>, BaseNode, SP<Node<Real>>>(m.attr("RealNode"));
    auto half = py::class_<Node<Half>, BaseNode, SP<Node<Half>>>(m.attr("HalfNode"));
    auto bf = py::class_<Node<BFloat16>, BaseNode, SP<Node<BFloat16>>>(m.attr("BFloat16Node"));
    bind_operators<Real>(real);
    bind_operators<Half>(half);
    bind_operators<BFloat16>(bf);
    auto integer = py::class_<Node<Int>, BaseNode, SP<Node<Int>>>(m.attr("IntNode"));
    bind_operators<Int>(integer);
  }
  // A Real data node converts to every scalar: Values(...).cast(ginn.Half) (ginn/node/data.h:100-108).
  py::class_<DataNode<Real>, Node<Real>, SP<DataNode<Real>>>(m.attr("RealDataNode"))
      .def("cast",
           [](const DataNode<Real>& n, Scalar_ s) -> py::object {
             switch (s) {
               case Scalar_::Real: return py::cast(cast_data<Real>(n));
               case Scalar_::Half: return py::cast(cast_data<Half>(n));
               case Scalar_::BFloat16: return py::cast(cast_data<BFloat16>(n));
               case Scalar_::Int: return py::cast(cast_data<Int>(n));
               default: return py::cast(cast_data<bool>(n));
             }
           })
      // values truncated to integers: labels that were read as floats (ginn-py/examples/mnist.py:38)
      .def("int", [](DataNode<Real>& n) {
        auto out = cast_data<Int>(n);
        out->set_has_grad(false);
        return out;
      })
      // conditions of Select (ginn-py/test/test_nodes.py:679)
      .def("bool", [](DataNode<Real>& n) {
        auto out = cast_data<bool>(n);
        out->set_has_grad(false);
        return out;
      });

  m.def("Data", [](const py::array& a) {
    auto n = Data<Real>(cpu());
    from_numpy<Real>(n->value(), a);
    n->set_has_grad(false);
    return SP<DataNode<Real>>(n.as_shared_ptr());
  });
  // Data(device, scalar), Data(device, shape, scalar), Data(shape, scalar) (ginn-py/node-py.cu.cpp:190-196)
  m.def("Data", &data_node, py::arg("device"), py::arg("shape"), py::arg("scalar") = Scalar_::Real);
  m.def("Data", [](const DevPtr& dev, Scalar_ s) { return data_node(dev, Shape{0}, s); }, py::arg("device"),
        py::arg("scalar") = Scalar_::Real);
  m.def("Data", [](const Shape& shape, Scalar_ s) { return data_node(cpu(), shape, s); }, py::arg("shape"),
        py::arg("scalar") = Scalar_::Real);
  // RealData(dev, shape), HalfData, ... (ginn-py/node-py.cu.cpp:181-188)
  m.def("RealData", [](const DevPtr& d, const Shape& s) { return data_node(d, s, Scalar_::Real); }, py::arg("dev"), py::arg("shape"));
  m.def("HalfData", [](const DevPtr& d, const Shape& s) { return data_node(d, s, Scalar_::Half); }, py::arg("dev"), py::arg("shape"));
  m.def("BFloat16Data", [](const DevPtr& d, const Shape& s) { return data_node(d, s, Scalar_::BFloat16); }, py::arg("dev"), py::arg("shape"));
  m.def("IntData", [](const DevPtr& d, const Shape& s) { return data_node(d, s, Scalar_::Int); }, py::arg("dev"), py::arg("shape"));
  m.def("BoolData", [](const DevPtr& d, const Shape& s) { return data_node(d, s, Scalar_::Bool); }, py::arg("dev"), py::arg("shape"));
  // lazily evaluated sizes (ginn-py/node/layout-py.cu.cpp:128-131)
  py::class_<DimNode, BaseNode, SP<DimNode>>(m, "DimNode").def_property_readonly("value", [](DimNode& d) { return d.value(); });
  m.def("Dim", [](Size n) { return SP<DimNode>(Dim(n).as_shared_ptr()); }, py::arg("dims"));
  m.def("Dim", [](const SP<BaseNode>& in, Size i) { return SP<DimNode>(Dim(BaseNodePtr(in), i).as_shared_ptr()); },
        py::arg("in"), py::arg("dim_idx"));
  // UpperTri(dev, size, scalar) (ginn-py/node/layout-py.cu.cpp:30-46,113-125)
  m.def("UpperTri",
        [](const DevPtr& dev, Size size, Scalar_ s) -> py::object {
          switch (s) {
            case Scalar_::Real: return py::cast(as_node(UpperTri<Real>(dev, size)));
            case Scalar_::Half: return py::cast(as_node(UpperTri<Half>(dev, size)));
            case Scalar_::BFloat16: return py::cast(as_node(UpperTri<BFloat16>(dev, size)));
            case Scalar_::Int: return py::cast(as_node(UpperTri<Int>(dev, size)));
            default: GINN_THROW("UpperTri exists for Real, Half, BFloat16 and Int");
          }
        },
        py::arg("dev"), py::arg("size"), py::arg("scalar") = Scalar_::Real);
  // Values(dev, nested list): a Real data node holding the literal (ginn/node/data.h:211-221)
  m.def("Values", [](const DevPtr& dev, const py::object& nested) {
    auto arr = py::array_t<Real, py::array::f_style | py::array::forcecast>::ensure(nested);
    if (!arr) throw std::invalid_argument("Values: a (nested) list of numbers is expected");
    auto n = Data<Real>(cpu());
    from_numpy<Real>(n->value(), arr);
    if (arr.ndim() == 0) n->value().resize(Shape{});
    n->move_to(dev);
    return SP<DataNode<Real>>(n.as_shared_ptr());
  }, py::arg("dev"), py::arg("values"));
  m.def("Values", [](const py::object& nested) {
    return py::module_::import("ginn").attr("Values")(SP<Device>(cpu()), nested);
  }, py::arg("values"));
  // Random(device, shape, scalar), Random(shape, scalar): uniform in [-1, 1] (ginn-py/node-py.cu.cpp:203-209)
  auto random_of = [](const DevPtr& dev, const Shape& shape, Scalar_ s) -> py::object {
    switch (s) {
      case Scalar_::Real: return py::cast(SP<DataNode<Real>>(Random<Real>(dev, shape).as_shared_ptr()));
      case Scalar_::Half: return py::cast(SP<DataNode<Half>>(Random<Half>(dev, shape).as_shared_ptr()));
      case Scalar_::BFloat16: return py::cast(SP<DataNode<BFloat16>>(Random<BFloat16>(dev, shape).as_shared_ptr()));
      default: throw std::invalid_argument("Random: a floating-point scalar is needed");
    }
  };
  m.def("Random", random_of, py::arg("device"), py::arg("shape"), py::arg("scalar") = Scalar_::Real);
  m.def("Random", [random_of](const Shape& shape, Scalar_ s) { return random_of(cpu(), shape, s); }, py::arg("shape"),
        py::arg("scalar") = Scalar_::Real);
  m.def("Weight",
        [](const DevPtr& dev, const Shape& shape, Scalar_ s) -> py::object {
          switch (s) {
            case Scalar_::Real: return py::cast(SP<WeightNode<Real>>(Weight<Real>(dev, shape).as_shared_ptr()));
            case Scalar_::Half: return py::cast(SP<WeightNode<Half>>(Weight<Half>(dev, shape).as_shared_ptr()));
            case Scalar_::BFloat16:
              return py::cast(SP<WeightNode<BFloat16>>(Weight<BFloat16>(dev, shape).as_shared_ptr()));
            default: throw std::invalid_argument("Weight: a floating-point scalar is needed");
          }
        },
        py::arg("device"), py::arg("shape"), py::arg("scalar") = Scalar_::Real);

  bind_float_nodes<Real>(m);
  bind_float_nodes<Half>(m);
  bind_float_nodes<BFloat16>(m);
  bind_shared_nodes<Int>(m);

  // ---- graphs ----
  py::class_<Graph>(m, "Graph")
      .def(py::init([](const SP<BaseNode>& sink) { return Graph(BaseNodePtr(sink)); }))
      .def("forward", [](Graph& g) { g.forward(); })
      .def("reset_forwarded", [](Graph& g) { g.reset_forwarded(); })
      .def("init_grad", [](Graph& g) { g.init_grad(); })
      .def("reset_grad", [](Graph& g) { g.reset_grad(); })
      .def("backward", [](Graph& g, double coeff) { g.backward(coeff); }, py::arg("loss_coeff") = 1.0)
      .def_property_readonly("size", [](const Graph& g) { return g.nodes().size(); })
      .def_property_readonly("sink", [](const Graph& g) -> py::object {
        SP<BaseNode> sink = g.sink().as_shared_ptr();
        if (auto r = std::dynamic_pointer_cast<Node<Real>>(sink)) return py::cast(r);
        if (auto h = std::dynamic_pointer_cast<Node<Half>>(sink)) return py::cast(h);
        if (auto b = std::dynamic_pointer_cast<Node<BFloat16>>(sink)) return py::cast(b);
        return py::cast(sink);
      });
  m.def("Autobatch", [](const Graph& g, bool gather) { return Autobatch(g, gather); }, py::arg("graph"),
        py::arg("gather") = false);
  py::class_<LevelExecutor>(m, "LevelExecutor")
      .def(py::init<const Graph&>(), py::keep_alive<1, 2>())
      .def("forward", [](LevelExecutor& e) { e.forward(); })
      .def("reset_forwarded", [](LevelExecutor& e) { e.reset_forwarded(); })
      .def("reset_grad", [](LevelExecutor& e) { e.reset_grad(); })
      .def("backward", [](LevelExecutor& e, double c) { e.backward(c); }, py::arg("loss_coeff") = 1.0)
      .def("freeze", [](LevelExecutor& e) { e.freeze(); })
      .def("fuse", [](LevelExecutor& e) { e.fuse(); })
      .def("thaw", [](LevelExecutor& e) { e.thaw(); })
      .def_property_readonly("launches", &LevelExecutor::launches)
      .def_property_readonly("levels", &LevelExecutor::levels);

  // ---- initialisers and updaters by scalar (ginn-py/init-py.cu.cpp, update-py.cu.cpp) ----
  m.def("Xavier", [](Scalar_ s) { return make_for<init::Xavier>(s); }, py::arg("scalar") = Scalar_::Real);
  m.def("Uniform", [](double range, Scalar_ s) { return make_for<init::Uniform>(s, static_cast<Real>(range)); },
        py::arg("range") = 1., py::arg("scalar") = Scalar_::Real);
  m.def("Sgd",
        [](double lr, double clip, Scalar_ s) {
          return make_for<update::Sgd>(s, static_cast<Real>(lr), static_cast<Real>(clip));
        },
        py::arg("lr") = 1e-1, py::arg("clip") = 5., py::arg("scalar") = Scalar_::Real);
  m.def("Adam",
        [](double lr, double clip, double eps, double b1, double b2, Scalar_ s) {
          return make_for<update::Adam>(s, static_cast<Real>(lr), static_cast<Real>(clip), static_cast<Real>(eps),
                                        static_cast<Real>(b1), static_cast<Real>(b2));
        },
        py::arg("lr") = 1e-3, py::arg("clip") = 5., py::arg("eps") = 1e-8, py::arg("beta_1") = 0.9,
        py::arg("beta_2") = 0.999, py::arg("scalar") = Scalar_::Real);
}
