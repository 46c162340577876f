"""The pybind11 module `ginn` (ginn_amd/python/ginn_py.cpp): the surface of the
reference's ginn-py that the product path needs.  CPU part: tensors and data
nodes exchanged with numpy, the text form, loud errors without a device (after
ginn-py/test/test_tensor.py).  GPU part: the training loop of
ginn-py/examples/mnist.py:62-92 on synthetic data against the CPU oracle."""
import numpy as np
import pytest

import ginn_amd
from conftest import rel_fro


@pytest.fixture(scope="module")
def ginn():
    return ginn_amd.pyginn()


def test_tensor_numpy_round_trip(ginn):
    a = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    t = ginn.RealTensor(ginn.cpu(), [1])
    t.set(a)
    assert t.shape == [2, 3, 4] and t.size == 24
    np.testing.assert_array_equal(t.numpy(), a)
    # storage is column-major: the first dimension runs fastest
    assert t.list()[:3] == [0.0, 12.0, 4.0]
    np.testing.assert_array_equal(t.m(), a.reshape(2, 12, order="F"))
    np.testing.assert_array_equal(t.v(), a.reshape(-1, order="F"))
    i = ginn.IntTensor(ginn.cpu(), [2, 2])
    i.set(np.array([[1, 2], [3, 4]], np.int32))
    assert i.list() == [1, 3, 2, 4]


def test_tensor_text_form(ginn):
    t = ginn.RealTensor(ginn.cpu(), [2, 1, 3])
    t.set(np.arange(1, 7, dtype=np.float32).reshape(2, 1, 3, order="F"))
    assert t.dumps() == "3\n2 1 3 \n1 2 3 4 5 6\n"
    u = ginn.RealTensor(ginn.cpu(), [0])
    u.loads(t.dumps())
    assert u.shape == [2, 1, 3]
    np.testing.assert_array_equal(u.numpy(), t.numpy())
    with pytest.raises(RuntimeError):
        u.loads("1\n3 \n1 2\n")


def test_data_and_weight_nodes(ginn):
    x = ginn.Data(np.array([[1.5, 2.0], [3.0, 4.0]]))
    assert x.shape == [2, 2] and not x.has_grad and x.dev.kind == ginn.DeviceKind.CPU
    assert x.int().value.list() == [1, 3, 2, 4]
    w = ginn.Weight(ginn.cpu(), [3, 2])
    assert w.has_grad and w.shape == [3, 2] and w.name.startswith("Weight")
    ginn.Uniform(0.5).init([w])
    assert np.abs(w.value.numpy()).max() <= 0.5
    w.has_grad = False
    assert not w.has_grad


def test_nodes_on_cpu_compute_or_fail_loudly(ginn):
    """The product-path nodes have host forms on cpu() (the same graph code as on the device); every other
    node refuses a cpu() tensor instead of computing something else."""
    x = ginn.Data(np.ones((2, 2)))
    s = ginn.Sigmoid(x)
    s.forward()
    assert s.value.list() == pytest.approx([1 / (1 + np.exp(-1.0))] * 4, rel=1e-6)
    W = ginn.Data(np.array([[1.0, 2.0], [3.0, 4.0]]))
    p = ginn.Prod(W, x)
    p.forward()
    assert p.value.list() == [3.0, 7.0, 3.0, 7.0]
    with pytest.raises(RuntimeError, match="HIP device only"):
        ginn.Variance(x).forward()


def test_devices_as_in_the_reference(ginn):
    """ginn-py/test/test_dev.py:29-106 on the CPU devices: a fresh Cpu() and the cpu() singleton are different
    devices with equal ids, an arena counts exactly the bytes of what lives on it (tensors of every scalar, the
    value and the empty gradient of a data node, the result of a node), clear() empties it."""
    d1 = ginn.Cpu()
    assert d1 == d1 and d1.id == d1.id and d1.precedence == 0
    d2 = ginn.PreallocCpu(100)
    assert d2.size == 100 and d1.id == d2.id and d2.precedence == 1 and d2.used == 0
    t = ginn.RealTensor(d2, [3], [1, 2, 3])
    assert d2.used == 12 and t.list() == [1, 2, 3]
    d2.clear()
    assert d2.used == 0
    t2, t3 = ginn.RealTensor(ginn.cpu(), [], [0]), ginn.RealTensor(ginn.cpu(), [], [0])
    assert t2.dev == t3.dev and t2.dev != d1
    assert ginn.cpu().kind == ginn.DeviceType.CPU and repr(d1.id) == "<DeviceId with kind: CPU, idx: 0>"
    for scalar, size in [(ginn.Real, 4), (ginn.Half, 2), (ginn.BFloat16, 2), (ginn.Int, 4), (ginn.Bool, 1)]:
        dev = ginn.PreallocCpu(100)
        t1 = ginn.Tensor(ginn.cpu(), [2, 3], scalar=scalar)
        assert dev.used == 0
        t2 = ginn.Tensor(dev, [1, 2], scalar=scalar)
        assert dev.used == t2.size * size
        ginn.Tensor(dev, scalar=scalar)
        assert dev.used == t2.size * size
        t4 = t2.copy_to(dev)
        assert dev.used == 2 * t2.size * size and t4.dev == dev
        t1.maybe_copy_to(dev)
        t1.move_to(dev)
        assert dev.used == (2 * t2.size + t1.size) * size
        t2.move_to(dev)  # already there
        assert dev.used == (2 * t2.size + t1.size) * size
    for Data, size in [(ginn.RealData, 4), (ginn.HalfData, 2)]:
        dev = ginn.PreallocCpu(100)
        x, y = Data(ginn.cpu(), [1, 2]), Data(ginn.cpu(), [1, 2])
        x.has_grad = False
        x.move_to(dev)
        assert dev.used == x.size * size
        y.move_to(dev)  # value and the (empty) gradient
        assert dev.used == 2 * x.size * size
        z = ginn.Add(x, y)
        g = ginn.Graph(z)
        assert dev.used == 2 * x.size * size
        g.forward()
        assert dev.used == 3 * x.size * size


def test_tensor_constructors_casts_and_views(ginn):
    """ginn-py/test/test_tensor.py: the constructor forms (:22-55), casts (:58-82), values and equality
    (:85-112), m() / v() as views that write through (:115-127), resizing through `shape` (:130-151)."""
    kinds = [(ginn.RealTensor, ginn.Real), (ginn.HalfTensor, ginn.Half), (ginn.IntTensor, ginn.Int),
             (ginn.BoolTensor, ginn.Bool), (ginn.BFloat16Tensor, ginn.BFloat16)]
    for cls, scalar in kinds:
        for t in (cls(), cls([2]), cls(ginn.cpu()), cls(ginn.cpu(), [2]), ginn.Tensor(scalar=scalar),
                  ginn.Tensor(scalar=scalar, shape=[2]), ginn.Tensor(device=ginn.cpu(), scalar=scalar),
                  ginn.Tensor(shape=[2], scalar=scalar, device=ginn.cpu())):
            assert t.scalar == scalar and all(t.scalar != other for _, other in kinds if other != scalar)
        t = cls(ginn.cpu())
        t.set([[1, 2, 3], [4, 5, 6]])
        assert t.real() == t.cast(ginn.Real) and t.int() == t.cast(ginn.Int)
        assert t.half() == t.cast(ginn.Half) and t.bool() == t.cast(ginn.Bool)
        assert t.cast(ginn.Real).scalar == ginn.Real and t.int().scalar == ginn.Int
    assert ginn.Tensor().scalar == ginn.Real and ginn.Tensor([2]).shape == [2]
    a, c, d = ginn.RealTensor(), ginn.RealTensor(), ginn.RealTensor()
    a.set([1, 2, 3])
    c.set([[1, 2, 3], [4, 5, 6]])
    d.set([[1, 2, 3], [4, 5, 6]])
    assert a.shape == [3] and c.shape == [2, 3] and a == a and a != c and c == d
    assert a.list() == [1, 2, 3] and c.list() == [1, 4, 2, 5, 3, 6]
    c.set_zero()
    assert c.list() == [0] * 6
    c.set_ones()
    assert c.list() == [1] * 6
    c.set_random()
    vals = c.list()
    assert all(-1 <= x <= 1 for x in vals) and all(x != y for x, y in zip(vals[:-1], vals[1:]))
    a = ginn.RealTensor([2, 3], [1, 2, 3, 4, 5, 6])
    np.testing.assert_array_equal(a.v(), np.array([1, 2, 3, 4, 5, 6], np.float32))
    np.testing.assert_array_equal(a.m(), np.array([[1, 3, 5], [2, 4, 6]], np.float32))
    v = a.v()
    v[3] = -4
    assert a.list() == [1, 2, 3, -4, 5, 6]
    m = a.m()
    m[0, 1] = -3
    assert a.list() == [1, 2, -3, -4, 5, 6]
    vals = [1, 2, 3, 4, 5, 6]
    a = ginn.RealTensor(ginn.cpu(), [2, 1, 3], vals)
    for shape in ([6], [3, 2]):
        a.shape = shape
        assert a.size == 6 and a.shape == shape and a.list() == vals
    for shape in ([4], [2, 2]):
        a.shape = shape
        assert a.size == 4 and a.shape == shape
    assert ginn.RealTensor([1], [2.5]).item() == 2.5


def test_keyword_forms_of_the_reference(ginn):
    """The argument names ginn-py gives its factories (ginn-py/node-py.cu.cpp:181-220, node/layout-py.cu.cpp,
    node/common-py.cu.cpp, node/weight-py.cu.cpp), as its tests call them (ginn-py/test/test_nodes.py:57, 76, 100,
    177, 216, 382, 942)."""
    dev = ginn.cpu()
    assert ginn.Random(dev, [3, 2, 1], scalar=ginn.Real).shape == [3, 2, 1]
    assert ginn.Random(device=dev, shape=[2, 2], scalar=ginn.Half).value.scalar == ginn.Half
    assert ginn.Random(shape=[4]).shape == [4]
    v = ginn.Values(values=[1, 2, 3, 4], dev=dev)
    assert v.value.list() == [1, 2, 3, 4] and ginn.Values(values=[[1, 2], [3, 4]]).shape == [2, 2]
    W = ginn.Values(dev, [[1, 2, 3, 4, 5, 6]])
    r = ginn.Reshape(W, shape=[3, 2])
    r.forward()
    assert r.shape == [3, 2]
    x = ginn.Values(dev, [[1, 2], [3, 4], [5, 6], [7, 8]])
    sl = ginn.Slice(x, offsets=[0, 1], sizes=[4, 1])
    ginn.Graph(sl).forward()
    assert sl.value.list() == [2, 4, 6, 8]
    ch = ginn.Chip(x, offset=2, dim=0)
    ginn.Graph(ch).forward()
    assert ch.value.list() == [5, 6]
    w = ginn.Weight(scalar=ginn.Real, device=dev, shape=[2, 3])
    assert w.shape == [2, 3] and w.copy(mode=ginn.Copy.Tied).shape == [2, 3]
    assert ginn.Data(dev, scalar=ginn.Half).value.scalar == ginn.Half
    assert ginn.Data([2, 3], scalar=ginn.Int).shape == [2, 3]
    assert ginn.Data(device=dev, shape=[2], scalar=ginn.Bool).value.scalar == ginn.Bool
    a, b, c = (ginn.Values(dev, [[1.0, 2.0]]) for _ in range(3))
    cpa = ginn.CwiseProdAdd(a, multiplicand=b, addend=c, multiplicand_bias=1.0)
    ginn.Graph(cpa).forward()
    assert cpa.value.list() == [3.0, 8.0]
    mask = ginn.Random(device=dev, shape=[2, 2]) * 0.5 + 1.0  # ginn-py/test/test_nodes.py check_grad's mask
    ginn.Graph(mask).forward()
    assert all(0.5 <= m <= 1.5 for m in mask.value.list())


def test_dim_nodes(ginn):
    """ginn-py/test/test_nodes.py:53-70 and the broadcasts that take a Dim (:334-335, 357-358), on cpu() where
    the broadcast is a view (extent 1) or refused loudly (a copy needs the device)."""
    x = ginn.Data(ginn.cpu(), [3, 2, 1])
    dims = [ginn.Dim(x, i) for i in range(3)]
    for d in dims:
        ginn.Graph(d).forward()
    assert [d.value for d in dims] == [3, 2, 1]
    assert ginn.Dim(7).value == 7
    a = ginn.Values(ginn.cpu(), [[1], [2], [3]])
    b = ginn.Values(ginn.cpu(), [[0.5, 1.5, 2.5]])
    same = ginn.ColBroadcast(a, ginn.Dim(b, 0))
    ginn.Graph(same).forward()
    assert same.shape == [3, 1] and same.value.list() == [1, 2, 3]


@pytest.mark.gpu
def test_mnist_style_training_loop(ginn):
    from oracle import nodes as N
    from oracle import update as U
    rng = np.random.default_rng(3)
    dimx, dimh, dimy, bs, lr = 64, 48, 10, 16, 1e-2
    dev = ginn.gpu()
    W, b = ginn.Weight(dev, [dimh, dimx]), ginn.Weight(dev, [dimh])
    V, c = ginn.Weight(dev, [dimy, dimh]), ginn.Weight(dev, [dimy])
    weights = [W, b, V, c]
    host = [rng.uniform(-0.3, 0.3, w.shape).astype(np.float32) for w in weights]
    for w, h in zip(weights, host):
        w.value.set(h)
    x_np = rng.uniform(0, 1, (dimx, bs)).astype(np.float32)
    y_np = rng.integers(0, dimy, (1, bs)).astype(np.float32)
    x, y = ginn.Data(x_np), ginn.Data(y_np).int()
    x.move_to(dev)
    y.move_to(dev)
    updater = ginn.Adam(lr)
    adam = U.Adam(lr=lr)
    ref = [h.copy() for h in host]
    for step in range(4):
        h = ginn.Sigmoid(ginn.Affine([W, x, b]))
        y_ = ginn.Affine([V, h, c])
        loss = ginn.Sum(ginn.PickNegLogSoftmax(y_, y))
        g = ginn.Graph(loss)
        g.forward()
        g.reset_grad()
        g.backward(1.0)
        want_loss, _, dWs, dbs = N.mlp_forward_backward(
            [N.SIGMOID, N.IDENTITY], [ref[0].astype(np.float64), ref[2].astype(np.float64)],
            [ref[1].astype(np.float64), ref[3].astype(np.float64)], x_np.astype(np.float64),
            y_np.reshape(-1).astype(np.int32))
        assert abs(loss.value.list()[0] - want_loss) <= 1e-4 * abs(want_loss)
        assert rel_fro(W.grad.numpy(), dWs[0]) <= 1e-4 and rel_fro(V.grad.numpy(), dWs[1]) <= 1e-4
        if step % 2:
            updater.update(weights)
        else:
            updater.update(g)
        for i, grad in enumerate([dWs[0], dbs[0], dWs[1], dbs[1]]):
            ref[i], _ = adam.update(ref[i], grad.astype(np.float32).reshape(ref[i].shape), i)
    for w, r in zip(weights, ref):
        assert rel_fro(w.value.numpy(), r) <= 1e-4
    # a weight listed twice gets two steps, one after the other (ginn/update/update.h:30-32)
    before = W.value.numpy().copy()
    W.grad.fill(0.25)
    sgd = ginn.Sgd(0.5, 5.0)
    sgd.update([W, W])
    np.testing.assert_allclose(W.value.numpy(), before - 2 * 0.5 * 0.25, rtol=0, atol=1e-6)
    # predictions as the example reads them: argmax over the rows of the output
    assert y_.value.maybe_copy_to(ginn.cpu()).m().shape == (dimy, bs)


@pytest.mark.gpu
def test_prod_nodes_and_autobatch_from_python(ginn):
    rng = np.random.default_rng(8)
    dev = ginn.gpu()
    a_np = rng.standard_normal((5, 4)).astype(np.float32)
    b_np = rng.standard_normal((4, 3)).astype(np.float32)
    a, b = ginn.Data(a_np), ginn.Data(b_np)
    a.move_to(dev)
    b.move_to(dev)
    a.has_grad = b.has_grad = True
    p = ginn.Prod(a, b)
    loss = ginn.Sum(ginn.Tanh(p))
    g = ginn.Graph(loss)
    g.forward()
    g.reset_grad()
    g.backward(1.0)
    want = a_np.astype(np.float64) @ b_np
    assert rel_fro(p.value.numpy(), want) <= 1e-4
    dp = 1 - np.tanh(want) ** 2
    assert rel_fro(a.grad.numpy(), dp @ b_np.T) <= 1e-4 and rel_fro(b.grad.numpy(), a_np.T @ dp) <= 1e-4
    # batched: per-slice products
    A = rng.standard_normal((3, 4, 6)).astype(np.float32)
    B = rng.standard_normal((4, 2, 6)).astype(np.float32)
    An, Bn = ginn.Data(A), ginn.Data(B)
    An.move_to(dev)
    Bn.move_to(dev)
    bp = ginn.BatchedProd(An, Bn)
    bp.forward()
    assert rel_fro(bp.value.numpy(), np.einsum("ikb,kjb->ijb", A.astype(np.float64), B)) <= 1e-4
    # Autobatch of two Affines sharing W, both merge forms, through the level executor
    W, bias = ginn.Weight(dev, [6, 4]), ginn.Weight(dev, [6])
    ginn.Xavier().init([W, bias])
    xs = [ginn.Data(rng.standard_normal((4, 1)).astype(np.float32)) for _ in range(3)]
    for xn in xs:
        xn.move_to(dev)
    outs = [ginn.Affine([W, xn, bias], nonlin="tanh") for xn in xs]
    total = ginn.Sum(ginn.Add(outs))
    g = ginn.Graph(total)
    g.forward()
    plain = total.value.list()[0]
    for gather in (False, True):
        g2 = ginn.Autobatch(g, gather=gather)
        ex = ginn.LevelExecutor(g2)
        ex.reset_forwarded()
        ex.forward()
        assert abs(g2.sink.value.list()[0] - plain) <= 1e-5 * max(1.0, abs(plain))
        assert g2.size != g.size


def test_scalars_tensors_and_casts(ginn):
    """Every scalar of ginn-py/tensor-py.h:36-48 (plus BFloat16): tensors exchange
    values with numpy, a Real data node casts to each of them."""
    a = np.array([[1.5, -2.0], [0.25, 4.0]])
    for name, cls in (("Half", ginn.HalfTensor), ("BFloat16", ginn.BFloat16Tensor)):
        t = cls(ginn.cpu(), [1])
        t.set(a)
        assert t.shape == [2, 2] and t.scalar == getattr(ginn, name)
        np.testing.assert_array_equal(np.asarray(t.numpy(), dtype=np.float64), a)  # exactly representable
    assert ginn.HalfTensor(ginn.cpu(), [2]).numpy().dtype == np.float16
    b = ginn.BoolTensor(ginn.cpu(), [1])
    b.set(np.array([[True, False], [False, True]]))
    assert b.list() == [True, False, False, True]
    x = ginn.Values(ginn.cpu(), [[1, 2, 3], [4, 5, 6]])
    assert x.shape == [2, 3] and x.value.list() == [1, 4, 2, 5, 3, 6]
    for scalar, cls in ((ginn.Real, "RealDataNode"), (ginn.Half, "HalfDataNode"), (ginn.BFloat16, "BFloat16DataNode"),
                        (ginn.Int, "IntDataNode"), (ginn.Bool, "BoolDataNode")):
        y = x.cast(scalar)
        assert type(y).__name__ == cls and y.shape == [2, 3]
        assert [float(v) for v in y.value.list()] == ([1.0] * 6 if scalar == ginn.Bool else [1, 4, 2, 5, 3, 6])
    w = ginn.Weight(scalar=ginn.Half, device=ginn.cpu(), shape=[2, 3])
    assert type(w).__name__ == "HalfWeightNode" and w.forwarded
    w.reset_forwarded()
    assert w.forwarded  # weights stay forwarded (ginn-py/test/test_nodes.py:945-948)
    w2 = w.copy(ginn.Copy.Tied)
    assert w2.id == w.id


@pytest.mark.gpu
@pytest.mark.parametrize("scalar_name", ["Real", "Half", "BFloat16"])
def test_reference_python_cases(ginn, scalar_name):
    """test_prod, test_batched_prod, test_affine, test_affine_w_broadcast and
    test_affine_w_high_rank of ginn-py/test/test_nodes.py:804-936, on the device,
    for Real and Half as there (Half eps 1e-2 / 2e-3) and for BFloat16."""
    scalar = getattr(ginn, scalar_name)
    dev = ginn.gpu()
    eps = {"Real": 1e-6, "Half": 1e-2, "BFloat16": 3e-2}[scalar_name]

    def check(a, b, eps):
        ginn.Graph(a).forward()
        ginn.Graph(b).forward()
        a_, b_ = a.value.maybe_copy_to(ginn.cpu()), b.value.maybe_copy_to(ginn.cpu())
        assert a_.shape == b_.shape
        assert a_.list() == pytest.approx(b_.list(), rel=eps, abs=eps * 1e-2)

    W = ginn.Values(dev, [[1, 2, 3], [4, 5, 6]]).cast(scalar)
    V = ginn.Values(dev, [[0.6, 0.5], [0.4, -0.1], [-0.2, -0.3]]).cast(scalar)
    WV = ginn.Values(dev, [[0.8, -0.6], [3.2, -0.3]]).cast(scalar)
    check(ginn.Prod(W, V), WV, eps)
    check(W * V, WV, eps)

    a = ginn.Random(dev, [2, 3, 4]).cast(scalar)
    b = ginn.Random(dev, [3, 5, 4]).cast(scalar)
    c = ginn.BatchedProd(a, b)
    for i in range(4):
        check(ginn.Chip(c, i, 2), ginn.Chip(a, i, 2) * ginn.Chip(b, i, 2), max(eps, 1e-5))

    Vc = ginn.Values(dev, [[0.6], [0.4], [-0.2]]).cast(scalar)
    bias = ginn.Values(dev, [[0.01], [0.02]]).cast(scalar)
    WVb = ginn.Values(dev, [[0.81], [3.22]]).cast(scalar)
    aeps = {"Real": 1e-6, "Half": 2e-3, "BFloat16": 2e-2}[scalar_name]
    check(ginn.Affine([W, Vc, bias]), WVb, aeps)
    check(W * Vc + bias, WVb, aeps)
    V2 = ginn.Values(dev, [[6, 5], [4, -1], [-2, -3]]).cast(scalar)
    b2 = ginn.Values(dev, [[0.1], [0.2]]).cast(scalar)
    check(ginn.Affine([W, V2, b2]), ginn.Values(dev, [[8.1, -5.9], [32.2, -2.8]]).cast(scalar), aeps)
    V3 = ginn.Values(dev, [[[6, 5], [6, 5]], [[4, -1], [4, -1]], [[-2, -3], [-2, -3]]]).cast(scalar)
    want = ginn.Values(dev, [[[8.1, -5.9], [8.1, -5.9]], [[32.2, -2.8], [32.2, -2.8]]]).cast(scalar)
    check(ginn.Affine([W, V3, b2]), want, aeps)
    # a few of the other nodes through the bindings
    check(ginn.AxisSum(V3, [0, 2]), ginn.Values(dev, [9.0, 9.0]).cast(scalar), aeps)
    check(1 - W, ginn.Values(dev, [[0, -1, -2], [-3, -4, -5]]).cast(scalar), aeps)
    lt = W < (W * 0 + 3.5)
    ginn.Graph(lt).forward()
    assert lt.value.list() == [True, False, True, False, True, False]
    # test_rank_view of ginn-py/test/test_nodes.py:183-201 and its neighbours Reshape / Slice
    M = ginn.Values(dev, [[1, 4], [2, 5], [3, 6]]).cast(scalar)
    check(ginn.RankView(M, 1), ginn.Values(dev, [1, 2, 3, 4, 5, 6]).cast(scalar), aeps)
    check(ginn.RankView(M, 2), M, aeps)
    check(ginn.RankView(M, 3), ginn.Values(dev, [[[1], [4]], [[2], [5]], [[3], [6]]]).cast(scalar), aeps)
    check(ginn.Slice(M, [1, 0], [2, 2]), ginn.Values(dev, [[2, 5], [3, 6]]).cast(scalar), aeps)


@pytest.mark.gpu
@pytest.mark.parametrize("scalar_name", ["Real", "Half"])
def test_reference_python_cases_of_the_other_nodes(ginn, scalar_name):
    """test_nonlin (:560-606), test_nonlin_extreme (:609-631), test_pick_and_friends (:634-672), test_axis_sum
    (:735-760), test_reduce (:771-784), test_weight (:940-962) and the Stack errors (:120-140) of
    ginn-py/test/test_nodes.py, forward, on the device, with the tolerances used there."""
    scalar = getattr(ginn, scalar_name)
    dev = ginn.gpu()
    half = scalar_name == "Half"

    def vals(v):
        return ginn.Values(dev, v).cast(scalar)

    def check(a, b, eps=1e-6):
        ginn.Graph(a).forward()
        ginn.Graph(b).forward()
        a_, b_ = a.value.maybe_copy_to(ginn.cpu()), b.value.maybe_copy_to(ginn.cpu())
        assert a_.shape == b_.shape
        eps = max(eps, 1e-3) if half else eps
        assert a_.list() == pytest.approx(b_.list(), rel=eps, abs=eps * 1e-1)

    W = vals([[-1, -2, -3], [4, 5, 6]])
    absW = vals([[1, 2, 3], [4, 5, 6]])
    check(ginn.Identity(W), W)
    check(ginn.Tanh(W), vals([[-0.76159415, -0.96402758, -0.99505475], [0.99932929, 0.99990920, 0.99998771]]))
    check(ginn.Relu(W), vals([[0, 0, 0], [4, 5, 6]]))
    check(ginn.Sigmoid(W), vals([[0.26894142, 0.11920292, 0.04742587], [0.98201379, 0.99330714, 0.99752737]]))
    check(ginn.Softmax(W), vals([[0.00669285, 9.11051194e-04, 1.23394576e-04],
                                 [0.99330715, 9.99088949e-01, 9.99876605e-01]]))
    check(ginn.Sqrt(ginn.CwiseProd(W, W)), absW)
    check(ginn.Log(absW), vals([[0, 0.69314718, 1.09861229], [1.38629436, 1.60943791, 1.79175947]]))
    x = vals([[10000.0], [-10000.0]])
    x2 = vals([[5.0], [-float("inf")]])
    check(ginn.Tanh(x), vals([[1], [-1]]))
    check(ginn.Sigmoid(x) + 1.0, vals([[1], [0]]) + 1.0)
    check(ginn.Softmax(ginn.Reshape(x, [1, 2])), ginn.Reshape(vals([[1], [1]]), [1, 2]))
    check(ginn.Softmax(x), vals([[1], [0]]))
    check(ginn.Softmax(x2), vals([[1], [0]]))

    P = vals([[-0.5, 0.55, -0.45], [1.0, 2.0, -1.0], [0.0, 0.0, 0.0], [0.3, -0.33, 1.3]])
    p, psm = vals([[0.3, 0.55, -1.0]]), vals([[0.23787436, 0.15987601, 0.06482681]])
    pnlsm = vals([[1.43601264, 1.8333567, 2.73603603]])
    il = [3, 0, 1]
    it = ginn.Values(dev, [3, 0, 1]).cast(ginn.Int)
    it.has_grad = False
    for idx in (il, it):
        check(ginn.Pick(P, idx), p)
        check(ginn.PickSoftmax(P, idx), psm)
        check(ginn.Pick(ginn.Softmax(P), idx), psm)
        check(ginn.PickNegLogSoftmax(P, idx), pnlsm)
        check(ginn.Pick(-ginn.Log(ginn.Softmax(P)), idx), pnlsm)
        check(-ginn.Log(ginn.Pick(ginn.Softmax(P), idx)), pnlsm)

    V = vals([[[1, 2, 3], [4, 5, 6]], [[0.1, 0.2, 0.3], [0.4, 0.5, 0.6]]])
    check(ginn.AxisSum(V, [0]), vals([[1.1, 2.2, 3.3], [4.4, 5.5, 6.6]]))
    check(ginn.AxisSum(V, [0, 1]), vals([5.5, 7.7, 9.9]))
    check(ginn.AxisSum(V, [0, 1, 2]), vals(23.1))
    check(ginn.AxisSum(V, [1]), vals([[5, 7, 9], [0.5, 0.7, 0.9]]))
    check(ginn.AxisSum(V, [1, 2]), vals([21, 2.1]))
    check(ginn.AxisSum(V, [2]), vals([[6, 15], [0.6, 1.5]]))
    check(ginn.AxisSum(V, [0, 2]), vals([6.6, 16.5]))
    for bad in ([0, 0], [2, 0]):
        with pytest.raises(RuntimeError):
            ginn.AxisSum(V, bad)
    M = vals([[1, 2, 3], [4, 5, 6]])
    check(ginn.Sum(M), vals(21))
    check(ginn.Mean(M), vals(3.5))
    check(ginn.Variance(M), vals(35.0 / 12.0))

    a, b, c, d = (vals([1 + 4 * i, 2 + 4 * i, 3 + 4 * i, 4 + 4 * i]) for i in range(4))
    e, f = vals([17, 18, 19]), vals([21, 22, 23, 24])
    for grid in ([[a, b], [c, d], [e, f]], [[a, b], [c, d], [e]], []):
        with pytest.raises(RuntimeError):
            ginn.Graph(ginn.Stack(grid)).forward()

    Wt = ginn.Weight(scalar=scalar, device=dev, shape=[2, 3])
    Wt.set_random()
    t = Wt.value.copy_to(dev)
    assert Wt.forwarded
    Wt.reset_forwarded()
    assert Wt.forwarded
    Wt.forward()
    assert Wt.value == t
    Wt.reset_grad()
    W2 = Wt.copy(ginn.Copy.Tied)
    assert W2.value is Wt.value and W2.grad is not Wt.grad
    W3 = Wt.copy(ginn.Copy.Deep)
    assert W3.value == Wt.value and W3.value is not Wt.value and W3.grad is not Wt.grad


@pytest.mark.gpu
def test_int_nodes_through_the_bindings(ginn):
    """The cases of ginn-py/test/test_nodes.py that run on ginn.Int (scalars3: Stack :73-118, test_add :388,
    test_add_scalar :416, test_subtract_scalar :434, test_prod_scalar :459, test_cwise_prod :476, CwiseProdAdd
    :490-545, test_cwise_max :547, test_reduce :793), on the device, with their known answers; integer
    arithmetic is exact, so values are compared for equality."""
    dev = ginn.gpu()
    I = ginn.Int

    def vals(v):
        return ginn.Values(dev, v).cast(I)

    def check(node, want):
        ginn.Graph(node).forward()
        got = node.value.maybe_copy_to(ginn.cpu())
        w = vals(want).value.maybe_copy_to(ginn.cpu())
        assert node.value.scalar == I
        assert got.shape == w.shape
        assert got.list() == w.list()

    a = vals([[1, 4], [2, 5], [3, 6]])
    b = vals([[-1, 4], [-2, 5], [-3, 6]])
    c = vals([[1, -4], [2, -5], [3, -6]])
    check(ginn.Add(a, b), [[0, 8], [0, 10], [0, 12]])
    check(a + b, [[0, 8], [0, 10], [0, 12]])
    check(ginn.Add([a, b, c]), [[1, 4], [2, 5], [3, 6]])
    check(a + b + a, [[1, 12], [2, 15], [3, 18]])
    check(ginn.AddScalar(a, 1), [[2, 5], [3, 6], [4, 7]])
    check(a + 1, [[2, 5], [3, 6], [4, 7]])
    check(1 + a, [[2, 5], [3, 6], [4, 7]])
    check(ginn.Subtract(a, b), [[2, 0], [4, 0], [6, 0]])
    check(ginn.SubtractScalar(1, a), [[0, -3], [-1, -4], [-2, -5]])
    check(1 - a, [[0, -3], [-1, -4], [-2, -5]])
    check(a - 1, [[0, 3], [1, 4], [2, 5]])
    check(-a, [[-1, -4], [-2, -5], [-3, -6]])
    check(ginn.ProdScalar(a, 2), [[2, 8], [4, 10], [6, 12]])
    check(2 * a, [[2, 8], [4, 10], [6, 12]])
    check(ginn.CwiseProd(a, b), [[-1, 16], [-4, 25], [-9, 36]])
    check(ginn.CwiseProdAdd(a, b, c), [[0, 12], [-2, 20], [-6, 30]])
    check(ginn.CwiseProdAdd(a, b, c, 1), [[1, 16], [0, 25], [-3, 36]])
    bv, cv = vals([-1, -2, -3]), vals([4, 5, 6])
    check(ginn.CwiseProdAdd(a, bv, cv), [[3, 0], [1, -5], [-3, -12]])
    check(ginn.CwiseProdAdd(a, bv, cv, 1), [[4, 4], [3, 0], [0, -6]])
    check(ginn.CwiseMax([b, c]), [[1, 4], [2, 5], [3, 6]])
    # Stack of rank-1 nodes
    parts = [vals([1 + 4 * i, 2 + 4 * i, 3 + 4 * i, 4 + 4 * i]) for i in range(6)]
    check(ginn.Stack([parts[0:2], parts[2:4], parts[4:6]]),
          [[[1, 5], [9, 13], [17, 21]], [[2, 6], [10, 14], [18, 22]], [[3, 7], [11, 15], [19, 23]],
           [[4, 8], [12, 16], [20, 24]]])
    check(ginn.RankView(a, 1), [1, 2, 3, 4, 5, 6])
    check(ginn.Reshape(a, [2, 3]), [[1, 3, 5], [2, 4, 6]])
    # comparison
    x, y = vals([[1], [2], [3], [4], [5]]), vals([[5], [4], [3], [2], [1]])
    lt = x < y
    ginn.Graph(lt).forward()
    assert lt.value.list() == [True, True, False, False, False]
    # selection (ginn-py/test/test_nodes.py:678-730); the fractions of the reference's case truncate to 0
    if_ = ginn.Values(dev, [[1, 0], [0, 1], [1, 0]]).bool()
    s1 = vals([[1, 2], [3, 4], [5, 6]])
    s2 = vals([[0.1, 0.2], [0.3, 0.4], [0.5, 0.6]])
    check(ginn.Select(if_, s1, s2), [[1, 0], [0, 4], [5, 0]])
    check(ginn.Select(if_, s1, 7), [[1, 7], [7, 4], [5, 7]])
    check(ginn.Select(if_, 7, s2), [[7, 0], [0, 7], [7, 0]])
    mask, mask2 = vals([[1, 0], [0, 1], [1, 0]]), vals([[1], [0], [1]])
    check(ginn.Mask(s1, mask, -1), [[1, -1], [-1, 4], [5, -1]])
    check(ginn.Mask(s1, mask2, 7), [[1, 2], [7, 7], [5, 6]])
    # axis orders (:245-300), broadcasts (:303-366), UpperTri (:369-385)
    t = vals([[[1, 2, 3, 4], [5, 6, 7, 8]], [[9, 10, 11, 12], [13, 14, 15, 16]],
              [[17, 18, 19, 20], [21, 22, 23, 24]]])
    tn = np.arange(1, 25).reshape(3, 2, 4)
    for perm in ([0, 2, 1], [2, 1, 0], [1, 0, 2], [1, 2, 0], [2, 0, 1], [0, 1, 2]):
        check(ginn.Permute(t, perm), tn.transpose(perm).tolist())
    check(ginn.Transpose(t, 2, 0), tn.transpose(2, 1, 0).tolist())
    col, row = vals([[1], [2], [3]]), vals([[0.1, 1.2, 2.3]])
    check(ginn.RowBroadcast(row, 3), [[0, 1, 2]] * 3)
    check(ginn.RowBroadcast(row, 1), [[0, 1, 2]])
    check(ginn.ColBroadcast(col, 3), [[1, 1, 1], [2, 2, 2], [3, 3, 3]])
    check(ginn.ColBroadcast(col, 1), [[1], [2], [3]])
    check(ginn.UpperTri(dev, 2, I), [[1, 1], [0, 1]])
    check(ginn.UpperTri(dev, 5, I), np.triu(np.ones((5, 5))).tolist())


@pytest.mark.gpu
@pytest.mark.parametrize("scalar_name", ["Half", "BFloat16"])
def test_mnist_style_training_loop_16bit(ginn, scalar_name):
    """The loop of ginn-py/examples/mnist.py:62-92 with 16-bit weights and
    activations (fp32 accumulation in the products): losses, gradients and
    weights follow the oracle within the 16-bit tolerance.  Plain gradient
    steps: Adam's step is +-lr whatever the size of a gradient, so an entry whose
    gradient is below the 16-bit rounding may legitimately move the other way."""
    from oracle import nodes as N
    from oracle import update as U
    scalar = getattr(ginn, scalar_name)
    rng = np.random.default_rng(11)
    dimx, dimh, dimy, bs, lr = 64, 48, 10, 16, 1e-2
    dev = ginn.gpu()
    shapes = [[dimh, dimx], [dimh], [dimy, dimh], [dimy]]
    weights = [ginn.Weight(dev, s, scalar) for s in shapes]
    host = []
    for w, s in zip(weights, shapes):
        w.value.set(rng.uniform(-0.3, 0.3, s))
        host.append(np.asarray(w.value.numpy(), dtype=np.float64))  # the values as stored
    W, b, V, c = weights
    x_np = rng.uniform(0, 1, (dimx, bs))
    y_np = rng.integers(0, dimy, (1, bs))
    x = ginn.Data(x_np)
    x.move_to(dev)
    xs = x.cast(scalar)
    x_np = np.asarray(xs.value.numpy(), dtype=np.float64)
    y = ginn.Data(y_np.astype(np.float32)).int()
    y.move_to(dev)
    assert type(ginn.Adam(lr, scalar=scalar)).__name__ == scalar_name + "Adam"
    updater = ginn.Sgd(0.1, 5.0, scalar=scalar)
    ref = [h.astype(np.float32) for h in host]
    for step in range(3):
        h = ginn.Sigmoid(ginn.Affine([W, xs, b]))
        loss = ginn.Sum(ginn.PickNegLogSoftmax(ginn.Affine([V, h, c]), y))
        g = ginn.Graph(loss)
        g.forward()
        g.reset_grad()
        g.backward(1.0)
        want_loss, _, dWs, dbs = N.mlp_forward_backward(
            [N.SIGMOID, N.IDENTITY], [ref[0].astype(np.float64), ref[2].astype(np.float64)],
            [ref[1].astype(np.float64), ref[3].astype(np.float64)], x_np, y_np.reshape(-1).astype(np.int32))
        assert abs(loss.value.list()[0] - want_loss) <= 2e-2 * abs(want_loss)
        assert rel_fro(np.asarray(W.grad.numpy(), np.float64), dWs[0]) <= 2e-2
        assert rel_fro(np.asarray(V.grad.numpy(), np.float64), dWs[1]) <= 2e-2
        updater.update(weights)
        for i, grad in enumerate([dWs[0], dbs[0], dWs[1], dbs[1]]):
            ref[i], _ = U.sgd_update(ref[i], grad.astype(np.float32).reshape(ref[i].shape), lr=0.1)
    for w, r in zip(weights, ref):
        assert rel_fro(np.asarray(w.value.numpy(), np.float64), r) <= 2e-2
