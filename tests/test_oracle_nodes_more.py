"""Pins oracle/nodes_more.py (the nodes around the product path) against the
reference's own known answers (test/nodes.cu.cpp, re-typed in
tests/golden/reference_nodes_more.json) and, for every backward formula,
against central finite differences with the reference's protocol
(test/testutil.h:93-171: delta 1e-4, random mask, expression evaluated as
e + e)."""
import json
from pathlib import Path

import numpy as np
import pytest

from conftest import farr
from oracle import nodes as N
from oracle import nodes_more as M


@pytest.fixture(scope="module")
def more():
    return json.loads((Path(__file__).parent / "golden" / "reference_nodes_more.json").read_text())


def approx(got, want, eps=1e-6):
    got, want = np.asarray(got, float), np.asarray(want, float)
    assert got.shape == want.shape, (got.shape, want.shape)
    assert (np.abs(got - want) <= eps * np.abs(want) + 1e-12).all(), (got, want)


def fd_check(f, inputs, analytic, rng, eps=1e-6):
    """Gradient of sum(mask * (f() + f())) w.r.t. every input by central
    differences, against 2 * analytic(mask)."""
    out = f()
    mask = np.asarray(rng.uniform(-1, 1, np.shape(out)))
    grads = analytic(mask)
    for x, g in zip(inputs, grads):
        if g is None:
            continue
        num = N.numeric_grad(lambda: f() + f(), x, mask)
        np.testing.assert_allclose(2 * np.asarray(g), num, rtol=1e-5, atol=eps)


# --- known answers -------------------------------------------------------------

def test_stack_goldens(more):
    for key in ("stack_rank1", "stack_rank2"):
        g = more[key]
        ins = [farr(x) for x in g["inputs"]]
        grid = [[ins[k] for k in row] for row in g["grid"]]
        approx(M.stack(grid), farr(g["expected"]))
    with pytest.raises(AssertionError):  # ragged input shapes (test/nodes.cu.cpp:113-124)
        M.stack([[farr([1., 2., 3., 4.]), farr([1., 2., 3.])]])


def test_chip_and_broadcast_goldens(more):
    g = more["chip"]
    x = farr(g["x"])
    approx(M.chip(x, 2, 0), farr(g["chip_2_0"]))
    approx(M.chip(x, 1, 1), farr(g["chip_1_1"]))
    g = more["broadcast"]
    a, b = farr(g["a"]), farr(g["b"])
    approx(M.row_broadcast(b, 3), farr(g["b3"]))
    approx(M.row_broadcast(b, 1), b)
    approx(np.repeat(a, 3, axis=1), farr(g["a3"]))  # ColBroadcast (already part of the product path)


def test_arithmetic_goldens(more):
    g = more["arith"]
    a, b, c = farr(g["a"]), farr(g["b"]), farr(g["c"])
    approx(a + b, farr(g["a_plus_b"]))
    approx(a + b + c, farr(g["a_plus_b_plus_c"]))
    approx(a + b + a, farr(g["a_plus_b_plus_a"]))
    approx(M.add_scalar(a, 1), farr(g["a_plus_1"]))
    approx(M.subtract(a, b), farr(g["a_minus_b"]))
    approx(M.subtract_scalar(1, a), farr(g["one_minus_a"]))
    approx(M.add_scalar(a, -1), farr(g["a_minus_1"]))
    approx(M.prod_scalar(a, -1), farr(g["neg_a"]))
    approx(M.prod_scalar(a, 2), farr(g["a_times_2"]))
    approx(a * b, farr(g["a_cwise_b"]))
    approx(N.cwise_prod_add_forward(a, b, c), farr(g["cwise_prod_add"]))
    approx(N.cwise_prod_add_forward(a, b, c, 1.0), farr(g["cwise_prod_add_bias1"]))
    bv, cv = farr(g["bvec"]), farr(g["cvec"])
    approx(N.cwise_prod_add_forward(a, bv, cv), farr(g["cwise_prod_add_bcast"]))
    approx(N.cwise_prod_add_forward(a, bv, cv, 1.0), farr(g["cwise_prod_add_bcast_bias1"]))
    approx(M.cwise_max([b, c]), farr(g["max_b_c"]))


def test_pick_goldens(more):
    g = more["pickles"]
    W, idx = farr(g["W"]), g["index"]
    approx(M.pick(W, idx), farr(g["pick"]))
    approx(M.pick_softmax(W, idx)[0], farr(g["pick_softmax"]), 1e-6)
    approx(M.pick(N.nonlin_forward(N.SOFTMAX, W), idx), farr(g["pick_softmax"]), 1e-6)
    approx(M.pick_neg_log_softmax(W, idx)[0], farr(g["pick_neg_log_softmax"]), 1e-6)
    approx(M.pick(-np.log(N.nonlin_forward(N.SOFTMAX, W)), idx), farr(g["pick_neg_log_softmax"]), 1e-6)
    # the fused head of oracle/nodes.py is the same function
    approx(N.pick_neg_log_softmax(W, np.array(idx))[0].reshape(1, -1), farr(g["pick_neg_log_softmax"]), 1e-6)
    g = more["pick_neg_log_sigmoid"]
    approx(M.pick_neg_log_sigmoid(farr(g["W"]), farr(g["p"]))[0], farr(g["expected"]), 1e-6)


def test_select_mask_compare_goldens(more):
    g = more["select"]
    cond, a, b = farr(g["if"]).astype(bool), farr(g["a"]), farr(g["b"])
    approx(M.select(cond, a, b), farr(g["y1"]))
    approx(M.select(cond, a, 7.0), farr(g["y2"]))
    approx(M.select(cond, 7.0, b), farr(g["y3"]))
    approx(M.select(cond, 7.0, -2.0), farr(g["y4"]))
    g = more["mask"]
    a = farr(g["a"])
    approx(M.mask(a, farr(g["mask"]), -1.0), farr(g["y1"]))
    approx(M.mask(a, farr(g["mask2"]), 7.0), farr(g["y2"]))
    g = more["comparison"]
    np.testing.assert_array_equal(M.less_than(farr(g["a"]), farr(g["b"])), farr(g["a_lt_b"]).astype(bool))


def test_sums_goldens(more):
    g = more["sums"]
    W, V = farr(g["W"]), farr(g["V"])
    approx(W.sum(), g["sum"])
    approx(M.mean(W), g["mean"])
    approx(M.variance(W)[0], g["variance"])
    approx(M.axis_sum(V, [0]), farr(g["V0"]))
    approx(M.axis_sum(V, [0, 1]), farr(g["V01"]))
    approx(M.axis_sum(V, [0, 1, 2]), g["V012"])
    approx(M.axis_sum(V, [1]), farr(g["V1"]))
    approx(M.axis_sum(V, [1, 2]), farr(g["V12"]))
    approx(M.axis_sum(V, [2]), farr(g["V2"]))
    approx(M.axis_sum(V, [0, 2]), farr(g["V02"]))
    for bad in ([0, 0], [2, 0]):
        with pytest.raises(AssertionError):
            M.axis_sum(V, bad)


def test_argmax_first_maximum_wins():
    x = farr([[1., 5., 5.], [7., 2., 7.]])
    np.testing.assert_array_equal(M.argmax_axis(x, 0), [1, 0, 1])
    np.testing.assert_array_equal(M.argmax_axis(x, 1), [1, 0])


# --- backward formulas by finite differences -----------------------------------------

def test_arithmetic_gradients():
    rng = np.random.default_rng(0)
    a, b, c = (np.asfortranarray(rng.uniform(-1, 1, (3, 2))) for _ in range(3))
    fd_check(lambda: M.subtract(a, b), [a, b], lambda m: M.subtract_backward(m), rng)
    fd_check(lambda: M.subtract_scalar(1.5, a), [a], lambda m: [-m], rng)
    fd_check(lambda: M.prod_scalar(a, -2.0), [a], lambda m: [-2.0 * m], rng)
    fd_check(lambda: M.cwise_max([a, b, c]), [a, b, c],
             lambda m: M.cwise_max_backward([a, b, c], M.cwise_max([a, b, c]), m), rng)
    mask = rng.uniform(0, 1, (3, 2)) >= 0.4
    fd_check(lambda: M.dropout_apply(a, mask, 0.4), [a], lambda m: [M.dropout_apply(m, mask, 0.4)], rng)


def test_select_and_mask_gradients():
    rng = np.random.default_rng(1)
    cond = rng.uniform(0, 1, (3, 2)) > 0.5
    a, b = np.asfortranarray(rng.uniform(-1, 1, (3, 2))), np.asfortranarray(rng.uniform(-1, 1, (3, 2)))
    fd_check(lambda: M.select(cond, a, b), [a, b], lambda m: M.select_backward(cond, a, b, m), rng)
    s = np.array(0.7)
    fd_check(lambda: M.select(cond, a, s), [a, s], lambda m: M.select_backward(cond, a, s, m), rng)
    fd_check(lambda: M.select(cond, s, b), [s, b], lambda m: M.select_backward(cond, s, b, m), rng)
    W = np.asfortranarray(rng.uniform(-1, 1, (2, 3, 2)))
    for ms in ((2, 3, 2), (2, 3, 1), (2, 1, 1)):  # the broadcast cases of test/nodes.cu.cpp:892-910
        msk = np.asfortranarray((rng.uniform(-1, 1, ms) > 0).astype(float))
        fd_check(lambda: M.mask(W, msk, 3.0), [W], lambda m: M.mask_backward(W, msk, m), rng)


def test_pick_gradients():
    rng = np.random.default_rng(2)
    W = np.asfortranarray(rng.uniform(-1, 1, (4, 3)))
    idx = [3, 0, 1]
    fd_check(lambda: M.pick(W, idx), [W], lambda m: M.pick_backward(W, idx, m), rng)
    fd_check(lambda: M.pick_softmax(W, idx)[0], [W],
             lambda m: M.pick_softmax_backward(W, idx, M.pick_softmax(W, idx)[1], m), rng)
    fd_check(lambda: M.pick_neg_log_softmax(W, idx)[0], [W],
             lambda m: M.pick_neg_log_softmax_backward(W, idx, M.pick_neg_log_softmax(W, idx)[1], m), rng)
    p = rng.integers(0, 2, (4, 3))
    fd_check(lambda: M.pick_neg_log_sigmoid(W, p)[0], [W],
             lambda m: M.pick_neg_log_sigmoid_backward(p, M.pick_neg_log_sigmoid(W, p)[1], m), rng)


def test_reduction_gradients():
    rng = np.random.default_rng(3)
    V = np.asfortranarray(rng.uniform(-1, 1, (2, 2, 3)))
    for axes in ([0], [0, 1], [0, 1, 2], [1], [1, 2], [2], [0, 2]):
        fd_check(lambda: M.axis_sum(V, axes), [V], lambda m: M.axis_sum_backward(V, axes, m), rng)
    fd_check(lambda: M.mean(V), [V], lambda m: M.mean_backward(V, m), rng)
    fd_check(lambda: M.variance(V)[0], [V], lambda m: M.variance_backward(V, M.variance(V)[1], m), rng)


def test_layout_gradients():
    rng = np.random.default_rng(4)
    ins = [np.asfortranarray(rng.uniform(-1, 1, (2, 2))) for _ in range(3)]
    for ids in ([[0, 1]], [[0, 1], [2, 0]], [[0, 0], [0, 0], [0, 0]]):
        used = sorted({k for row in ids for k in row})
        fd_check(lambda: M.stack([[ins[k] for k in row] for row in ids]), [ins[k] for k in used],
                 lambda m: [M.stack_backward(ids, 3, m)[k] for k in used], rng)
    x = np.asfortranarray(rng.uniform(-1, 1, (4, 2, 3)))
    for off, dim in ((3, 0), (0, 1), (1, 2), (2, 2)):
        fd_check(lambda: M.chip(x, off, dim), [x], lambda m: M.chip_backward(x, off, dim, m), rng)
    b = np.asfortranarray(rng.uniform(-1, 1, (1, 3)))
    fd_check(lambda: M.row_broadcast(b, 3), [b], lambda m: M.row_broadcast_backward(m), rng)
    fd_check(lambda: M.transpose(x, 0, 2)[0], [x], lambda m: [N.permute_backward(m, M.transpose(x, 0, 2)[1])], rng)


def test_inplace_cwise_prod_backward_equals_plain():
    rng = np.random.default_rng(5)
    a, b = rng.uniform(0.5, 1.5, (2, 3, 2)), rng.uniform(0.5, 1.5, (2, 3, 2))
    dy = rng.uniform(-1, 1, (2, 3, 2))
    da, db = M.inplace_cwise_prod_backward(a * b, b, dy)
    np.testing.assert_allclose(da, dy * b)
    np.testing.assert_allclose(db, dy * a, rtol=1e-12)
