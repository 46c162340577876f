"""The nodes around the product path on the HIP device -- arithmetic, selection,
picking, reductions, layout and in-place nodes of the host layer -- against
oracle/nodes_more.py, through the C++ host layer (tests/cpp/zoo_shim.cpp) and
with the reference's protocol (test/check_node.h:27-121): the expression is
evaluated as e = f() + f(), the loss is Sum(mask * e).  Also the reference's
known answers (test/nodes.cu.cpp) straight on the device, dropout statistics
(test/dropoutnodes.cu.cpp), argmax and the device-side random fill."""
import ctypes
import json
from pathlib import Path

import numpy as np
import pytest

from conftest import farr, rel_fro
from ginn_amd import capi
from oracle import nodes as N
from oracle import nodes_more as M

pytestmark = pytest.mark.gpu

DTYPES = [capi.F32, capi.F16, capi.BF16]
SHIM = Path(__file__).resolve().parent / "cpp" / "libhost_shim.so"
FP = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def shim():
    if not SHIM.exists():
        pytest.fail(f"{SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(SHIM))
    lib.zoo_last_error.restype = ctypes.c_char_p
    lib.zoo_expect_throw.restype = ctypes.c_char_p
    return lib


@pytest.fixture(scope="module")
def more():
    return json.loads((Path(__file__).parent / "golden" / "reference_nodes_more.json").read_text())


def f32(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float32))


def fptr(a):
    return a.ctypes.data_as(FP)


def run(shim, name, dt, inputs, has_grad=None, ip=(), fp=(), index=(), mask=None, out_shape=()):
    """Calls shim_zoo; returns (value, grads)."""
    n = len(inputs)
    has_grad = list(has_grad) if has_grad is not None else [1] * n
    ins = [f32(x) for x in inputs]
    dims = [d for x in ins for d in x.shape]
    out = np.zeros(out_shape, np.float32, order="F")
    grads = [np.zeros(x.shape, np.float32, order="F") for x in ins]
    ipa = (ctypes.c_int * max(1, len(ip)))(*ip)
    fpa = (ctypes.c_float * max(1, len(fp)))(*fp)
    idx = np.ascontiguousarray(np.asarray(index, dtype=np.int32).reshape(-1, order="F"))
    maskp = fptr(f32(mask)) if mask is not None else None
    rc = shim.shim_zoo(name.encode(), dt, n, (ctypes.c_long * max(1, len(dims)))(*dims),
                       (ctypes.c_int * max(1, n))(*[x.ndim for x in ins]), (FP * max(1, n))(*[fptr(x) for x in ins]),
                       (ctypes.c_int * max(1, n))(*has_grad), ipa, fpa,
                       idx.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), idx.size, maskp, fptr(out),
                       (FP * max(1, n))(*[fptr(g) for g in grads]))
    assert rc == 0, shim.zoo_last_error().decode()
    return out, grads


def rnd(rng, shape, dt, lo=-1.0, hi=1.0):
    from gpu_util import round_to
    return round_to(rng.uniform(lo, hi, shape), dt)


# name, input shapes, ip, fp, index maker, forward(ins, idx) -> value, backward(ins, idx, value, dy) -> grads
def _cases():
    c = []

    def add(name, shapes, fwd, bwd, ip=(), fp=(), index=None, has_grad=None, positive=False):
        c.append(dict(name=name, shapes=shapes, fwd=fwd, bwd=bwd, ip=ip, fp=fp, index=index, has_grad=has_grad,
                      positive=positive))

    s32 = (3, 2)
    add("subtract", [s32, s32], lambda x, i: M.subtract(*x), lambda x, i, v, dy: M.subtract_backward(dy))
    add("subtract_op", [s32, s32], lambda x, i: M.subtract(*x), lambda x, i, v, dy: M.subtract_backward(dy))
    add("scalar_minus", [s32], lambda x, i: M.subtract_scalar(1.5, x[0]), lambda x, i, v, dy: [-dy], fp=[1.5])
    add("minus_scalar", [s32], lambda x, i: M.add_scalar(x[0], -0.75), lambda x, i, v, dy: [dy], fp=[0.75])
    add("plus_scalar", [s32], lambda x, i: M.add_scalar(x[0], 0.5), lambda x, i, v, dy: [dy], fp=[0.5])
    add("scalar_plus", [s32], lambda x, i: M.add_scalar(x[0], 0.5), lambda x, i, v, dy: [dy], fp=[0.5])
    add("times_scalar", [s32], lambda x, i: M.prod_scalar(x[0], -2.0), lambda x, i, v, dy: [-2 * dy], fp=[-2.0])
    add("scalar_times", [s32], lambda x, i: M.prod_scalar(x[0], 3.0), lambda x, i, v, dy: [3 * dy], fp=[3.0])
    add("neg", [s32], lambda x, i: -x[0], lambda x, i, v, dy: [-dy])
    add("add3", [s32] * 3, lambda x, i: x[0] + x[1] + x[2], lambda x, i, v, dy: [dy, dy, dy])
    add("add_repeat", [s32] * 2, lambda x, i: 2 * x[0] + x[1], lambda x, i, v, dy: [2 * dy, dy])
    add("cwise_max", [(5, 4)] * 3, lambda x, i: M.cwise_max(x), lambda x, i, v, dy: M.cwise_max_backward(x, v, dy))
    cond = lambda rng, shp: rng.integers(0, 2, shp)
    add("select_nn", [(4, 3)] * 2, lambda x, i: M.select(i, x[0], x[1]),
        lambda x, i, v, dy: M.select_backward(i, x[0], x[1], dy), index=lambda rng: cond(rng, (4, 3)))
    add("select_ns", [(4, 3)], lambda x, i: M.select(i, x[0], 7.0),
        lambda x, i, v, dy: M.select_backward(i, x[0], np.array(7.0), dy)[:1], fp=[7.0],
        index=lambda rng: cond(rng, (4, 3)))
    add("select_sn", [(4, 3)], lambda x, i: M.select(i, 7.0, x[0]),
        lambda x, i, v, dy: M.select_backward(i, np.array(7.0), x[0], dy)[1:], fp=[7.0],
        index=lambda rng: cond(rng, (4, 3)))
    for ms in ((2, 3, 2), (2, 3, 1), (2, 1, 1)):
        add("mask", [(2, 3, 2), ms], lambda x, i: M.mask(x[0], x[1], 3.0),
            lambda x, i, v, dy: M.mask_backward(x[0], x[1], dy) + [None], fp=[3.0], has_grad=[1, 0])
        add("inplace_mask", [(2, 3, 2), ms], lambda x, i: M.mask(x[0], x[1], -3.0),
            lambda x, i, v, dy: M.mask_backward(x[0], x[1], dy) + [None], fp=[-3.0], has_grad=[1, 0])
    pidx = lambda rng: rng.integers(0, 6, 5)
    add("pick", [(6, 5)], lambda x, i: M.pick(x[0], i), lambda x, i, v, dy: M.pick_backward(x[0], i, dy), index=pidx)
    add("pick_vec", [(6, 5)], lambda x, i: M.pick(x[0], i), lambda x, i, v, dy: M.pick_backward(x[0], i, dy),
        index=pidx)
    add("pick_softmax", [(6, 5)], lambda x, i: M.pick_softmax(x[0], i)[0],
        lambda x, i, v, dy: M.pick_softmax_backward(x[0], i, M.pick_softmax(x[0], i)[1], dy), index=pidx)
    add("pick_of_softmax", [(6, 5)], lambda x, i: M.pick_softmax(x[0], i)[0],
        lambda x, i, v, dy: M.pick_softmax_backward(x[0], i, M.pick_softmax(x[0], i)[1], dy), index=pidx)
    add("pick_nls", [(6, 5)], lambda x, i: M.pick_neg_log_softmax(x[0], i)[0],
        lambda x, i, v, dy: M.pick_neg_log_softmax_backward(x[0], i, M.pick_neg_log_softmax(x[0], i)[1], dy),
        index=pidx)
    add("neg_log_pick_softmax", [(6, 5)], lambda x, i: M.pick_neg_log_softmax(x[0], i)[0],
        lambda x, i, v, dy: M.pick_neg_log_softmax_backward(x[0], i, M.pick_neg_log_softmax(x[0], i)[1], dy),
        index=pidx)
    add("pick_nlsig", [(4, 3)], lambda x, i: M.pick_neg_log_sigmoid(x[0], i)[0],
        lambda x, i, v, dy: M.pick_neg_log_sigmoid_backward(i, M.pick_neg_log_sigmoid(x[0], i)[1], dy),
        index=lambda rng: cond(rng, (4, 3)))
    for off, dim in ((3, 0), (0, 1), (1, 2), (2, 2)):
        add("chip", [(4, 2, 3)], lambda x, i, off=off, dim=dim: M.chip(x[0], off, dim),
            lambda x, i, v, dy, off=off, dim=dim: M.chip_backward(x[0], off, dim, dy), ip=[off, dim])
    for axes in ([0], [0, 1], [0, 1, 2], [1], [1, 2], [2], [0, 2]):
        add("axis_sum", [(2, 2, 3)], lambda x, i, axes=axes: M.axis_sum(x[0], axes),
            lambda x, i, v, dy, axes=axes: M.axis_sum_backward(x[0], axes, dy), ip=[len(axes)] + axes)
    add("axis_sum", [(33, 17, 5, 3)], lambda x, i: M.axis_sum(x[0], [1, 3]),
        lambda x, i, v, dy: M.axis_sum_backward(x[0], [1, 3], dy), ip=[2, 1, 3])
    add("variance", [(7, 9)], lambda x, i: M.variance(x[0])[0],
        lambda x, i, v, dy: M.variance_backward(x[0], M.variance(x[0])[1], dy))
    add("mean", [(7, 9)], lambda x, i: M.mean(x[0]), lambda x, i, v, dy: M.mean_backward(x[0], dy))
    for ids in ([[0, 1]], [[0, 1], [2, 0]], [[0, 0], [0, 0], [0, 0]], [[0, 1], [2, 3], [4, 5]]):
        k = max(max(r) for r in ids) + 1
        add("stack", [(3, 2)] * k, lambda x, i, ids=ids: M.stack([[x[q] for q in r] for r in ids]),
            lambda x, i, v, dy, ids=ids, k=k: M.stack_backward(ids, k, dy), ip=[len(ids), len(ids[0])],
            index=lambda rng, ids=ids: np.array(ids).reshape(-1))
    add("row_broadcast", [(1, 5)], lambda x, i: M.row_broadcast(x[0], 4),
        lambda x, i, v, dy: M.row_broadcast_backward(dy), ip=[4])
    add("row_broadcast_dim", [(1, 5), (3, 2)], lambda x, i: M.row_broadcast(x[0], 3),
        lambda x, i, v, dy: M.row_broadcast_backward(dy) + [None], ip=[0], has_grad=[1, 0])
    add("transpose", [(4, 2, 3)], lambda x, i: M.transpose(x[0], 0, 2)[0],
        lambda x, i, v, dy: [N.permute_backward(dy, [2, 1, 0])], ip=[0, 2])
    add("inplace_add", [s32] * 3, lambda x, i: x[0] + x[1] + x[2], lambda x, i, v, dy: [dy, dy, dy])
    add("inplace_add_repeat", [s32] * 2, lambda x, i: x[0] + 2 * x[1], lambda x, i, v, dy: [dy, 2 * dy])
    add("inplace_add_scalar", [s32], lambda x, i: M.add_scalar(x[0], 3.14), lambda x, i, v, dy: [dy], fp=[3.14])
    add("inplace_prod_scalar", [s32], lambda x, i: M.prod_scalar(x[0], -5.0), lambda x, i, v, dy: [-5 * dy],
        fp=[-5.0])
    add("inplace_cwise_prod", [(2, 3, 2)] * 2, lambda x, i: x[0] * x[1],
        lambda x, i, v, dy: M.inplace_cwise_prod_backward(v, x[1], dy), positive=True)
    add("inplace_sigmoid", [s32], lambda x, i: N.nonlin_forward(N.SIGMOID, x[0]),
        lambda x, i, v, dy: [N.nonlin_backward(N.SIGMOID, dy, x[0], v)])
    add("inplace_layernorm", [(16, 5)], lambda x, i: N.layernorm_forward(x[0])[0],
        lambda x, i, v, dy: [M.layernorm_backward_assign(dy, v, N.layernorm_forward(x[0])[1])])
    add("inplace_permute", [(4, 2, 3)], lambda x, i: N.permute(x[0], [2, 0, 1]),
        lambda x, i, v, dy: [N.permute_backward(dy, [2, 0, 1])], ip=[3, 2, 0, 1])
    add("inplace_dropout_p0", [s32], lambda x, i: x[0], lambda x, i, v, dy: [dy])
    add("dropout_p1", [s32], lambda x, i: 0 * x[0], lambda x, i, v, dy: [0 * dy])
    return c


CASES = _cases()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("case", range(len(CASES)), ids=[f"{i}-{c['name']}" for i, c in enumerate(CASES)])
def test_node_against_oracle(shim, dt, case):
    from gpu_util import TOL, round_to
    c = CASES[case]
    rng = np.random.default_rng(1000 + case)
    lo = 0.5 if c["positive"] else -1.0
    ins = [rnd(rng, s, dt, lo, 1.5 if c["positive"] else 1.0) for s in c["shapes"]]
    if c["name"] in ("mask", "inplace_mask"):
        ins[1] = (ins[1] > 0).astype(np.float32)
    if c["name"] == "cwise_max":  # keep the maxima unique beyond the 16-bit rounding
        ins = [round_to(x + 0.25 * k, dt) for k, x in enumerate(ins)]
    idx = c["index"](rng) if c["index"] else np.zeros(0, np.int32)
    ins64 = [x.astype(np.float64) for x in ins]
    want = np.asarray(c["fwd"](ins64, idx), dtype=np.float64)
    mask = round_to(rng.uniform(-1, 1, want.shape), dt) if want.ndim else round_to(np.array(rng.uniform(-1, 1)), dt)
    value, grads = run(shim, c["name"], dt, ins, c["has_grad"], c["ip"], c["fp"], idx, mask=mask.reshape(want.shape),
                       out_shape=want.shape)
    want_g = c["bwd"](ins64, idx, want, mask.astype(np.float64).reshape(want.shape))
    tol = TOL[dt] * (1 if dt == capi.F32 else 2)
    assert rel_fro(value, 2 * want) <= tol, c["name"]
    for k, g in enumerate(want_g):
        if g is None:
            continue
        assert rel_fro(grads[k], 2 * np.asarray(g)) <= 3 * tol, (c["name"], k)


@pytest.mark.parametrize("dt", DTYPES)
def test_reference_known_answers_on_the_device(shim, more, dt):
    """The forward goldens of test/nodes.cu.cpp for these nodes, computed on the
    device (plain forward, no doubling)."""
    eps = {capi.F32: 1e-6, capi.F16: 2e-3, capi.BF16: 2e-2}[dt]

    def check(name, inputs, want, **kw):
        want = farr(want) if not np.isscalar(want) else np.array(float(want))
        got, _ = run(shim, name, dt, [farr(x, np.float32) for x in inputs], out_shape=want.shape, **kw)
        np.testing.assert_allclose(got, want, rtol=eps, atol=eps)

    g = more["arith"]
    a, b, c = g["a"], g["b"], g["c"]
    check("subtract", [a, b], g["a_minus_b"])
    check("subtract_op", [a, b], g["a_minus_b"])
    check("scalar_minus", [a], g["one_minus_a"], fp=[1.0])
    check("minus_scalar", [a], g["a_minus_1"], fp=[1.0])
    check("plus_scalar", [a], g["a_plus_1"], fp=[1.0])
    check("scalar_plus", [a], g["a_plus_1"], fp=[1.0])
    check("neg", [a], g["neg_a"])
    check("times_scalar", [a], g["a_times_2"], fp=[2.0])
    check("scalar_times", [a], g["a_times_2"], fp=[2.0])
    check("add3", [a, b, c], g["a_plus_b_plus_c"])
    check("add_repeat", [a, b], g["a_plus_b_plus_a"])
    check("cwise_prod", [a, b], g["a_cwise_b"])
    check("cwise_max", [b, c], g["max_b_c"])
    for key in ("stack_rank1", "stack_rank2"):
        s = more[key]
        check("stack", s["inputs"], s["expected"], ip=[3, 2], index=np.array(s["grid"]).reshape(-1))
    s = more["chip"]
    check("chip", [s["x"]], s["chip_2_0"], ip=[2, 0])
    check("chip", [s["x"]], s["chip_1_1"], ip=[1, 1])
    s = more["broadcast"]
    check("row_broadcast", [s["b"]], s["b3"], ip=[3])
    check("row_broadcast", [s["b"]], s["b"], ip=[1])
    check("row_broadcast_dim", [s["b"], s["a"]], s["b3"], ip=[0])
    check("row_broadcast_dim", [s["b"], s["a"]], s["b"], ip=[1])
    check("col_broadcast", [s["a"]], s["a3"], ip=[3])
    s = more["pickles"]
    pe = {capi.F32: 1e-6, capi.F16: 1e-3, capi.BF16: 1e-2}[dt]
    for name, key in (("pick", "pick"), ("pick_vec", "pick"), ("pick_softmax", "pick_softmax"),
                      ("pick_of_softmax", "pick_softmax"), ("pick_nls", "pick_neg_log_softmax"),
                      ("neg_log_pick_softmax", "pick_neg_log_softmax")):
        got, _ = run(shim, name, dt, [farr(s["W"], np.float32)], index=s["index"], out_shape=(1, 3))
        np.testing.assert_allclose(got, farr(s[key]), rtol=max(pe, eps), atol=eps)
    s = more["pick_neg_log_sigmoid"]
    check("pick_nlsig", [s["W"]], s["expected"], index=farr(s["p"], np.int32))
    s = more["select"]
    cond = farr(s["if"], np.int32)
    check("select_nn", [s["a"], s["b"]], s["y1"], index=cond)
    check("select_ns", [s["a"]], s["y2"], fp=[7.0], index=cond)
    check("select_sn", [s["b"]], s["y3"], fp=[7.0], index=cond)
    check("select_ss", [], s["y4"], fp=[7.0, -2.0], ip=[2, 3, 2], index=cond)
    s = more["mask"]
    check("mask", [s["a"], s["mask"]], s["y1"], fp=[-1.0])
    check("mask", [s["a"], s["mask2"]], s["y2"], fp=[7.0])
    s = more["sums"]
    check("sum", [s["W"]], s["sum"])
    check("mean", [s["W"]], s["mean"])
    check("variance", [s["W"]], s["variance"])
    for axes, key in (([0], "V0"), ([0, 1], "V01"), ([0, 1, 2], "V012"), ([1], "V1"), ([1, 2], "V12"), ([2], "V2"),
                      ([0, 2], "V02")):
        check("axis_sum", [s["V"]], s[key], ip=[len(axes)] + axes)
    s = more["comparison"]
    check("less_than", [s["a"], s["b"]], s["a_lt_b"])
    check("constant_like", [s["a"]], [[2.5]] * 5, fp=[2.5])
    check("ones_like", [s["a"]], [[1.0]] * 5)


@pytest.mark.parametrize("dt", [capi.F32, capi.F16])
@pytest.mark.parametrize("inplace", [0, 1])
@pytest.mark.parametrize("p", [0.0, 0.25, 0.5, 0.75, 1.0])
def test_dropout_statistics(shim, dt, inplace, p):
    """test/dropoutnodes.cu.cpp:30-106: on all-ones input the mean of the output
    is 1 within 1e-2 (values are 0 or 1 / (1 - p)), p = 0 keeps everything, p = 1
    drops everything; the backward pass uses the very mask of the forward pass;
    a second forward pass draws another mask."""
    n = 2_000_000
    y = np.zeros(n, np.float32)
    dx = np.zeros(n, np.float32)
    differs = ctypes.c_int(-1)
    rc = shim.shim_dropout(dt, inplace, ctypes.c_float(p), ctypes.c_long(n), fptr(y), fptr(dx), ctypes.byref(differs))
    assert rc == 0, shim.zoo_last_error().decode()
    if p == 0.0:
        assert (y == 1).all() and (dx == 1).all()
    elif p == 1.0:
        assert (y == 0).all()
        # the in-place node leaves the gradient alone when p = 1, as the reference's does
        # (ginn/node/inplace.h:135-140 guards its rescaling with p < 1)
        assert (dx == (1 if inplace else 0)).all()
    else:
        from gpu_util import round_to
        keep = float(round_to(np.array([1.0 / (1.0 - p)]), dt)[0])
        assert set(np.unique(y)) == {0.0, keep}
        assert abs(y.mean() - 1.0) <= 1e-2
        np.testing.assert_array_equal(dx, y)  # same mask, same scale, dy = 1
        assert differs.value == 1
        # neighbouring elements are independent: P(both kept) = (1 - p)^2
        both = ((y[:-1] != 0) & (y[1:] != 0)).mean()
        assert abs(both - (1 - p) ** 2) <= 5e-3


@pytest.mark.parametrize("dt", DTYPES)
def test_argmax(shim, dt):
    from gpu_util import round_to
    rng = np.random.default_rng(5)
    x = round_to(rng.uniform(-1, 1, (6, 5, 4)), dt)
    x[2, 1, 3] = x[4, 1, 3] = 2.0  # a tie: the first one wins
    for dim in (0, 1, 2):
        want = M.argmax_axis(x, dim)
        out = np.zeros(want.shape, np.int64, order="F")
        rc = shim.shim_argmax(dt, (ctypes.c_long * 3)(*x.shape), 3, fptr(f32(x)), dim,
                              out.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)))
        assert rc == 0, shim.zoo_last_error().decode()
        np.testing.assert_array_equal(out, want)
    flat = np.zeros(1, np.int64)
    shim.shim_argmax(dt, (ctypes.c_long * 3)(*x.shape), 3, fptr(f32(x)), -1,
                     flat.ctypes.data_as(ctypes.POINTER(ctypes.c_longlong)))
    assert flat[0] == int(np.argmax(x.reshape(-1, order="F")))


@pytest.mark.parametrize("dt", DTYPES)
def test_device_side_random_fill(shim, dt):
    """Tensor::set_random on a GPU tensor (ginn/tensor.h:446-470): uniform in
    [-1, 1], another stream per call; mean 0 and variance 1/3 within sampling error."""
    n = 1_000_000
    a, b = np.zeros(n, np.float32), np.zeros(n, np.float32)
    rc = shim.shim_random(dt, ctypes.c_long(n), fptr(a), fptr(b))
    assert rc == 0, shim.zoo_last_error().decode()
    for v in (a, b):
        assert v.min() >= -1.0 and v.max() <= 1.0
        assert abs(v.mean()) <= 5e-3
        assert abs(v.var() - 1.0 / 3.0) <= 5e-3
    assert (a != b).mean() > 0.9
    assert abs(np.corrcoef(a, b)[0, 1]) <= 5e-3
    assert abs(np.corrcoef(a[:-1], a[1:])[0, 1]) <= 5e-3


def test_error_paths_of_these_nodes(shim):
    expect = {0: "Input shapes mismatch", 1: "Inner container sizes mismatch", 2: "empty()",
              3: "empty()", 4: "uniquely", 5: "sorted", 6: "Dropout probability", 7: "Dropout probability",
              8: "Index size does not match", 9: "offset_"}
    for which, text in expect.items():
        msg = shim.zoo_expect_throw(which).decode()
        assert text in msg, (which, msg)
