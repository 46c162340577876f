"""Gradients that reset_grad() flags instead of zeroing (BaseNode::GradUse in
ginn_amd/ginn/node.h).  The reference zeroes every gradient in reset_grad()
(ginn/node.h:218-222) and adds in every backward pass; a gradient with one
user that can overwrite is only flagged here and the user overwrites it (a
product runs with beta = 0).  The gradients must not depend on that: one graph
with every overwriting node as a sole user (attention block, gated product,
vocabulary head; tests/cpp/lazy_shim.cpp) is run with the flagging on and off,
node by node and through the level executor in every mode, over several passes."""
import ctypes
import math
from pathlib import Path

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi

pytestmark = pytest.mark.gpu

SHIM = Path(__file__).resolve().parent / "cpp" / "libhost_shim.so"
MODES = {"graph": 0, "executor": 1, "frozen": 2, "chained": 3, "recorded": 4}


@pytest.fixture(scope="module")
def shim():
    if not SHIM.exists():
        pytest.fail(f"{SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(SHIM))
    lib.lazy_last_error.restype = ctypes.c_char_p
    return lib


def fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def run(lib, dt, lazy, mode, passes, hs=16, nh=2, B=3, T=24, V=40, seed=0):
    from gpu_util import round_to
    C = hs * nh
    rng = np.random.default_rng(seed)
    shapes = [(C, C), (C,), (C, C), (C,), (C, C), (C,), (C, C), (C, C), (V, C), (V,)]
    params = [np.asfortranarray(round_to(rng.uniform(-1, 1, s) / math.sqrt(C), dt).astype(np.float32)) for s in shapes]
    x = np.asfortranarray(round_to(rng.uniform(-1, 1, (C, B, T)), dt).astype(np.float32))
    targets = rng.integers(0, V, B * T).astype(np.int32)
    grads = [np.zeros(s, np.float32, order="F") for s in shapes]
    dx = np.zeros((C, B, T), np.float32, order="F")
    loss = np.zeros(1, np.float32)
    flagged = ctypes.c_long(-1)
    fills = ctypes.c_long(-1)
    pp = (ctypes.POINTER(ctypes.c_float) * 10)(*[fptr(p) for p in params])
    gp = (ctypes.POINTER(ctypes.c_float) * 10)(*[fptr(g) for g in grads])
    rc = lib.shim_lazy_graph(dt, lazy, MODES[mode], passes, hs, nh, B, T, V, fptr(x),
                             targets.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), pp, fptr(loss), fptr(dx), gp,
                             ctypes.byref(flagged), ctypes.byref(fills))
    assert rc == 0, lib.lazy_last_error().decode()
    return loss[0], dx, grads, flagged.value, fills.value


@pytest.mark.parametrize("dt", [capi.F32, capi.F16, capi.BF16])
@pytest.mark.parametrize("mode", list(MODES))
def test_flagged_gradients_equal_zeroed_ones(shim, dt, mode):
    """Same loss and gradients with and without the flagging, after three passes
    (a stale flag or a gradient that was neither zeroed nor overwritten would
    show as last pass's gradient added in, or as zeros)."""
    want_loss, want_dx, want_grads, none, _ = run(shim, dt, 0, "graph", 1)
    assert none == 0
    got_loss, got_dx, got_grads, flagged, fills = run(shim, dt, 1, mode, 3)
    # 19 float nodes of the graph have a single user that overwrites (directly or
    # through views and in-place nodes); none of them needed a fill on demand.
    assert flagged >= 15, flagged
    assert fills == 0, fills
    # beta = 0 instead of 0 + 1 * x changes no rounding; the split of a long sum
    # over workgroups may differ between the two launches of a product.
    # 16-bit storage: the executor adds the users of one gradient in another order than the node-by-node
    # pass does, which moves a result by one unit of the last place (2^-11 for f16, 2^-8 for bf16).
    tol = {capi.F32: 1e-6, capi.F16: 2e-3, capi.BF16: 1e-2}[dt]
    assert abs(got_loss - want_loss) <= tol * max(1.0, abs(want_loss))
    assert np.abs(want_dx).max() > 0
    assert rel_fro(got_dx, want_dx) <= tol
    for g, w in zip(got_grads, want_grads):
        assert np.abs(w).max() > 0
        assert rel_fro(g, w) <= tol


@pytest.mark.parametrize("mode", list(MODES))
def test_switch_off_matches_in_every_mode(shim, mode):
    """set_lazy_grad_reset(false): nothing is flagged and every mode still
    agrees with the node-by-node pass."""
    want_loss, want_dx, want_grads, _, _ = run(shim, capi.F32, 0, "graph", 1, seed=3)
    got_loss, got_dx, got_grads, flagged, fills = run(shim, capi.F32, 0, mode, 2, seed=3)
    assert flagged == 0 and fills == 0
    assert rel_fro(got_dx, want_dx) <= 1e-6
    for g, w in zip(got_grads, want_grads):
        assert rel_fro(g, w) <= 1e-6


def test_reading_a_flagged_gradient_gives_zeros(shim):
    out = np.full(1, -1, np.float32)
    assert shim.shim_lazy_semantics(0, fptr(out)) == 0, shim.lazy_last_error().decode()
    assert out[0] == 0.0


def test_graphs_that_share_a_node(shim):
    """Two graphs over one product node, reset one after the other, run one after
    the other: the first user overwrites, the second adds (ginn/node.h:237-254
    accumulates over both)."""
    out = np.zeros(1, np.float32)
    assert shim.shim_lazy_semantics(1, fptr(out)) == 0, shim.lazy_last_error().decode()
    assert out[0] == pytest.approx(1 - math.tanh(4.0) ** 2 + 3.0, rel=1e-6)


def test_only_single_overwriting_users_qualify(shim):
    out = np.zeros(1, np.float32)
    assert shim.shim_lazy_semantics(2, fptr(out)) == 0, shim.lazy_last_error().decode()
    # A, B (Prod overwrites), Sum(P) and Sum(Q) (Add overwrites); not P (three
    # uses), not Q (Sum adds to its input), not the sink.
    assert out[0] == 4


@pytest.mark.parametrize("dt", [capi.F32, capi.BF16])
@pytest.mark.parametrize("mode", ["graph", "executor", "frozen", "recorded"])
def test_weight_gradients_beside_the_pass_are_the_same_bits(shim, dt, mode):
    """Products of >= 1 GFLOP into the gradients of weights run on the GPU's second stream while a
    backward pass runs (internal::BesidePass in ginn_amd/ginn/node.h; the reference has one stream,
    ginn/dev.h:188-189), and so do the bias row sums of Affines without an activation from 2^20
    elements on (ginn_amd/ginn/node/affine.h).  Same kernels on the same operands: after three passes
    without a wait in between, loss and every gradient are bit-identical to the run on one stream."""
    sizes = dict(hs=64, nh=12, B=4, T=512, V=1024)  # 768 x 768 x 2048 products: 2.4 GFLOP; 768 x 2048 row sums
    try:
        shim.shim_set_beside_pass(0)
        want_loss, want_dx, want_grads, _, _ = run(shim, dt, 1, mode, 3, seed=11, **sizes)
        shim.shim_set_beside_pass(1)
        got_loss, got_dx, got_grads, _, _ = run(shim, dt, 1, mode, 3, seed=11, **sizes)
    finally:
        shim.shim_set_beside_pass(1)
    assert got_loss == want_loss
    np.testing.assert_array_equal(got_dx, want_dx)
    for g, w in zip(got_grads, want_grads):
        assert np.abs(w).max() > 0
        np.testing.assert_array_equal(g, w)


@pytest.mark.parametrize("mode", ["graph", "executor", "frozen"])
def test_a_weight_with_several_gradient_writers_stays_on_the_pass_stream(shim, mode):
    """A product goes to the second stream only when its target has one gradient writer in the pass
    (internal::BesidePass): the second stream is not ordered against what the pass enqueues later.
    W feeds a 2.1 GFLOP product, a narrow product and an Add, so all three writers of dW stay on the
    pass's stream; V feeds one 2.1 GFLOP product, which goes beside.  Loss and both gradients are
    bit-identical to the run on one stream."""
    d = 1024
    rng = np.random.default_rng(5)
    w, v, x1 = (np.asfortranarray(rng.uniform(-1, 1, (d, d)).astype(np.float32) / math.sqrt(d)) for _ in range(3))
    x2 = np.asfortranarray(rng.uniform(-1, 1, (d, 8)).astype(np.float32))

    def once(beside):
        dw = np.zeros((d, d), np.float32, order="F")
        dv = np.zeros((d, d), np.float32, order="F")
        loss = np.zeros(1, np.float32)
        n = ctypes.c_long(-1)
        shim.shim_set_beside_pass(beside)
        rc = shim.shim_shared_weight_graph(MODES[mode], d, fptr(w), fptr(v), fptr(x1), fptr(x2), fptr(loss),
                                           fptr(dw), fptr(dv), ctypes.byref(n))
        assert rc == 0, shim.lazy_last_error().decode()
        return loss[0], dw, dv, n.value

    try:
        want_loss, want_dw, want_dv, none = once(0)
        got_loss, got_dw, got_dv, beside = once(1)
    finally:
        shim.shim_set_beside_pass(1)
    assert none == 0
    assert beside == 3  # dV of each of the three passes; never dW
    assert np.abs(want_dw).max() > 0 and np.abs(want_dv).max() > 0
    assert got_loss == want_loss
    np.testing.assert_array_equal(got_dw, want_dw)
    np.testing.assert_array_equal(got_dv, want_dv)


@pytest.mark.parametrize("which", [0, 1, 2, 3])
def test_in_place_steps_have_run_when_forward_returns(shim, which):
    """InPlaceProdScalar / InPlaceMask overwrite their input in forward() in the reference
    (ginn/node/inplace.h:104-123, 152-212).  Here they may wait for their first reader (a Softmax takes
    them over); whoever holds the node they write over must still see the final contents once
    Graph::forward() / LevelExecutor::forward() has returned, also when nobody read their value."""
    rng = np.random.default_rng(which)
    a = np.asfortranarray(rng.uniform(-1, 1, (3, 4)).astype(np.float32))
    b = np.asfortranarray(rng.uniform(-1, 1, (4, 2)).astype(np.float32))
    mask = np.asfortranarray(np.array([[1, 0], [1, 1], [0, 1]], np.float32))
    out = np.zeros((3, 2), np.float32, order="F")
    assert shim.shim_inplace_semantics(which, fptr(a), fptr(b), fptr(mask), fptr(out)) == 0, shim.lazy_last_error().decode()
    want = np.where(mask != 0, np.float32(0.5) * (a.astype(np.float64) @ b).astype(np.float32), np.float32(-5))
    np.testing.assert_allclose(out, want, rtol=1e-6, atol=1e-7)


def test_a_skipped_backward_does_not_leak_into_the_next_pass(shim):
    """A fused Softmax backward tells the in-place steps below to skip theirs; when their backward never
    runs in that pass, the next pass (which needs them) gives what a fresh graph gives."""
    rng = np.random.default_rng(9)
    a = np.asfortranarray(rng.uniform(-1, 1, (3, 4)).astype(np.float32))
    b = np.asfortranarray(rng.uniform(-1, 1, (4, 2)).astype(np.float32))
    mask = np.asfortranarray(np.array([[1, 0], [1, 1], [0, 1]], np.float32))
    out = np.zeros(12, np.float32)
    assert shim.shim_inplace_semantics(4, fptr(a), fptr(b), fptr(mask), fptr(out)) == 0, shim.lazy_last_error().decode()
    assert np.abs(out[6:]).max() > 0
    assert (out[6:].reshape(3, 2, order="F")[mask == 0] == 0).all()  # masked entries pass no gradient
    np.testing.assert_array_equal(out[:6], out[6:])


@pytest.mark.parametrize("dt", [capi.F32, capi.BF16, capi.F16])
@pytest.mark.parametrize("mode", [0, 1, 2, 3])
@pytest.mark.parametrize("read", [0, 1])
@pytest.mark.parametrize("hs,nh,B,T", [(64, 4, 8, 64), (16, 2, 3, 24), (64, 8, 16, 256)])
def test_batched_products_on_permuted_views(shim, dt, mode, read, hs, nh, B, T):
    """Permute nodes between projections and batched products (the heads of an attention layer,
    examples/min-gpt.cu.cpp:117-135) copy nothing: BatchedProd reads the slices where the projection wrote
    them, writes its result where the next node reads it, and the gradients take the same ways back
    (ginn_amd/ginn/node/slices.h).  Values and gradients against numpy fp64, node by node and through the level
    executor, frozen and recorded; the input changes between the passes, so a frozen pass that replayed a
    value instead of computing it would differ; with `read` the postponed values are asked for mid-pass.
    The 64-row heads in 16 bit take the one-launch two-level kernel, the others run level by level."""
    from gpu_util import TOL, round_to
    if T == 256 and (mode != 3 or read or dt == capi.F32):
        pytest.skip("the large case checks the one-launch kernel and the launch count of a recorded pass")
    C, N = hs * nh, B * T
    rng = np.random.default_rng(hs + T + mode)
    x1 = np.asfortranarray(round_to(rng.uniform(-1, 1, (C, N)), dt))
    x2 = np.asfortranarray(round_to(rng.uniform(-1, 1, (C, N)), dt))
    W = [np.asfortranarray(round_to(rng.uniform(-1, 1, (C, C)) / math.sqrt(C), dt)) for _ in range(3)]
    mask = np.asfortranarray(round_to(rng.uniform(-1, 1, (C, N)), dt))
    y = np.zeros((C, N), np.float32, order="F")
    dx = np.zeros((C, N), np.float32, order="F")
    dW = [np.zeros((C, C), np.float32, order="F") for _ in range(3)]
    k_out = np.zeros((T, hs, B, nh), np.float32, order="F")
    s_out = np.zeros((T, T, B, nh), np.float32, order="F")
    kernels = ctypes.c_long(-1)
    rc = shim.shim_permuted_products(dt, mode, read, hs, nh, B, T, fptr(x1), fptr(x2),
                                     (ctypes.POINTER(ctypes.c_float) * 3)(*[fptr(w) for w in W]), fptr(mask), fptr(y),
                                     fptr(dx), (ctypes.POINTER(ctypes.c_float) * 3)(*[fptr(g) for g in dW]),
                                     fptr(k_out), fptr(s_out), ctypes.byref(kernels))
    assert rc == 0, shim.lazy_last_error().decode()
    # numpy fp64 on x2: projections [hs, nh, B, T]; s[t, u, b, h] = sum_e K[e,h,b,t] Q[e,h,b,u]; y = V s
    X, Wk, Wq, Wv, M = (a.astype(np.float64) for a in (x2, W[0], W[1], W[2], mask))
    heads = lambda P: P.reshape((hs, nh, B, T), order="F")
    K, Q, V = heads(Wk @ X), heads(Wq @ X), heads(Wv @ X)
    S = np.einsum("ehbt,ehbu->tubh", K, Q)
    Y = np.einsum("ehbt,tubh->ehbu", V, S)
    dY = heads(M)
    dV = np.einsum("ehbu,tubh->ehbt", dY, S)
    dS = np.einsum("ehbt,ehbu->tubh", V, dY)
    dK = np.einsum("tubh,ehbu->ehbt", dS, Q)
    dQ = np.einsum("tubh,ehbt->ehbu", dS, K)
    flat = lambda P: P.reshape((C, N), order="F")
    want_dW = [flat(dK) @ X.T, flat(dQ) @ X.T, flat(dV) @ X.T]
    want_dx = Wk.T @ flat(dK) + Wq.T @ flat(dQ) + Wv.T @ flat(dV)
    tol = 4 * TOL[dt]
    assert rel_fro(y, flat(Y)) <= tol
    assert rel_fro(dx, want_dx) <= tol
    for got, want in zip(dW, want_dW):
        assert rel_fro(got, want) <= tol
    if read:
        assert rel_fro(k_out, np.transpose(K, (3, 0, 2, 1))) <= tol
        assert rel_fro(s_out, S) <= tol
    if mode == 3 and T == 256:
        # three projections, two batched products, the element-wise product and the sum forward; backward
        # the broadcast, the product with the mask, four batched products and six projections' products
        # (those of the weights with their split-K folds) plus the fills of reset_grad: 28 launches, none of
        # them a copy for one of the four Permute nodes (8 more, forward and backward, with the copies)
        assert 0 < kernels.value <= 30, kernels.value
