// The level executor's host logic on a recording stand-in for the device
// library (null_abi.py): which launches a small graph turns into.  Prints one
// line per phase: "<phase>: <call> <count>, ..." for the multi_* calls, the
// number of table uploads, and the number of launches nodes made themselves.
#include <cstdio>
#include <cstring>
#include <sstream>
#include <string>
#include <vector>

#include <ginn/ginn.h>

extern "C" const char* null_abi_log(void);
extern "C" void null_abi_clear(void);

using namespace ginn;

static void report(const char* phase) {
  std::istringstream in(null_abi_log());
  std::string name;
  long count;
  std::string tables;
  int uploads = 0, direct = 0;
  while (in >> name >> count) {
    if (name.rfind("ginn_hip_multi_", 0) == 0)
      tables += (tables.empty() ? "" : ", ") + name.substr(9) + " " + std::to_string(count);
    else if (name == "ginn_hip_memcpy_h2d")
      ++uploads;
    else if (name != "ginn_hip_sync" && name != "ginn_hip_ctx_stream" && name != "ginn_hip_ctx_device")
      ++direct;
  }
  std::printf("%s: [%s] uploads=%d direct=%d\n", phase, tables.c_str(), uploads, direct);
  null_abi_clear();
}

int main() {
  auto dev = gpu();
  // Level 1: tanh, sigmoid, relu of x and relu of z (four operations of three
  // kinds and two lengths); level 2: two products and an N-ary add; level 3:
  // the sum of everything.  b = Tanh(x) has two users on level 2.
  auto x = Random(dev, {8, 5});
  auto z = Random(dev, {3, 7});
  x->set_has_grad(true);
  z->set_has_grad(true);
  auto a = Sigmoid(x);
  auto b = Tanh(x);
  auto c = Relu(x);
  auto zz = Relu(z);
  auto p = CwiseProd(a, b);
  auto q = CwiseProd(b, c);
  auto s = Add(p, q, c);
  auto five = Add(s, s, s, s, s);  // five users of s.grad() on one level: a reduction
  auto loss = Sum(CwiseProd(five, five)) + Sum(zz);
  null_abi_clear();

  Graph g(loss);
  LevelExecutor ex(g);
  std::printf("levels: %zu nodes: %zu\n", ex.levels(), g.nodes().size());
  ex.reset_forwarded();
  ex.forward();
  report("forward 1");
  ex.reset_grad();
  report("reset 1");
  ex.backward(1.);
  report("backward 1");
  const size_t built = ex.rebuilt();
  ex.reset_forwarded();
  ex.forward();
  ex.reset_grad();
  ex.backward(1.);
  report("pass 2");
  std::printf("rebuilt in pass 2: %zu\n", ex.rebuilt() - built);
  ex.freeze();
  ex.reset_forwarded();
  ex.forward();
  ex.reset_grad();
  ex.backward(1.);
  report("frozen pass");
  std::printf("rebuilt frozen: %zu\n", ex.rebuilt() - built);
  // fuse(): levels 1..5 of the forward pass have no self-running node between
  // them: one chain launch; everything that depends on x is one chain, Relu(z) another.
  ex.fuse();
  null_abi_clear();  // the chain tables were uploaded
  ex.forward();
  report("fused forward");
  ex.reset_grad();
  report("fused reset");
  ex.backward(1.);
  report("fused backward");
  std::printf("chain launches built: %zu\n", ex.chains());
  ex.thaw();
  // plain execution of the same graph: every node launches for itself
  g.reset_forwarded();
  g.forward();
  g.reset_grad();
  g.backward(1.);
  report("plain pass");

  // A leaf whose gradient gets a reduction on two levels (a bias added in two layers, five
  // columns each): level by level these are two reductions of five sources; a frozen executor
  // sums all ten at the end of the backward pass.
  {
    auto bias = Random(dev, {8});
    bias->set_has_grad(true);
    std::vector<NodePtr<Real>> tops;
    for (int i = 0; i < 5; ++i) {
      auto xi = Random(dev, {8});
      auto lower = Add(NodePtr<Real>(xi), NodePtr<Real>(bias));
      tops.push_back(Add(NodePtr<Real>(Tanh(NodePtr<Real>(lower))), NodePtr<Real>(bias)));
    }
    Graph two(Sum(NodePtr<Real>(Add(tops))));
    LevelExecutor ex2(two);
    ex2.reset_forwarded();
    ex2.forward();
    ex2.reset_grad();
    null_abi_clear();
    ex2.backward(1.);
    report("two-level backward");
    ex2.freeze();
    ex2.forward();
    ex2.reset_grad();
    null_abi_clear();
    ex2.backward(1.);
    report("two-level backward frozen");
  }

  // Autobatch (ginn/autobatch.h:42-202): six Affines that share W on one
  // height and two that share it on the next become two merged products.
  {
    auto W = Random(dev, {4, 3});
    auto bias = Random(dev, {4});
    auto U = Random(dev, {3, 4});
    auto ub = Random(dev, {3});
    std::vector<NodePtr<Real>> tops;
    for (int i = 0; i < 6; ++i) {
      auto xi = Random(dev, {3, 1});
      auto h = Affine<TanhOp>(W, xi, bias);
      if (i < 2) tops.push_back(Affine<SigmoidOp>(U, h, ub));
      else tops.push_back(Sum(h));
    }
    std::vector<NodePtr<Real>> sums;
    for (auto& t : tops) sums.push_back(Sum(t));
    Graph before(Add(sums));
    before.forward();  // the rewrite reads operand shapes
    auto count = [](const Graph& gr, const char* what) {
      size_t n = 0;
      for (auto& node : gr.nodes()) n += node->name() == what;
      return n;
    };
    Graph after = Autobatch(before);
    std::printf("autobatch: affines %zu -> %zu, prods %zu -> %zu\n", count(before, "AffineNode"),
                count(after, "AffineNode"), count(before, "Prod"), count(after, "Prod"));
    std::printf("autobatch glue: RowwiseCat %zu RowwiseUncat %zu\n", count(after, "RowwiseCat"), count(after, "RowwiseUncat"));
  }
  return 0;
}
