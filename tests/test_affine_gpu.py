"""GPU parity of the AffineNode entry points (ginn_hip_affine_fwd,
ginn_hip_affine_bwd_pre) and of the stand-alone nonlinearities against the
numpy node oracle, which itself is pinned to the reference's golden vectors
(tests/test_oracle_nodes.py).  Known answers from test/nodes.cu.cpp:1117-1200
are checked directly as well."""
import ctypes

import numpy as np
import pytest

from conftest import farr, rel_fro
from ginn_amd import capi
from oracle import nodes as N

pytestmark = pytest.mark.gpu

DTYPES = [capi.F32, capi.F16, capi.BF16]
ACTS = [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.GELU, N.GELU2, N.SOFTMAX]


@pytest.fixture(scope="module")
def dev():
    from gpu_util import Dev
    d = Dev()
    yield d
    d.close()


def affine_fwd(dev, dt, act, ins, want_pre):
    """Runs ginn_hip_affine_fwd on ins = [W0, X0, W1, X1, ..., bias] (fp32 numpy,
    already rounded to dt).  Returns (Y, pre or None)."""
    pairs = (len(ins) - 1) // 2
    m = ins[0].shape[0]
    n = int(np.prod(ins[1].shape[1:]))
    bufs, Wp, Xp, ks = [], [], [], []
    for p in range(pairs):
        W, X = ins[2 * p], ins[2 * p + 1]
        bw, pw, _ = dev.put(W, dt)
        bx, px, _ = dev.put(X.reshape(X.shape[0], -1, order="F"), dt)
        bufs += [bw, bx]
        Wp.append(pw)
        Xp.append(px)
        ks.append(W.shape[1])
    bb, pb, _ = dev.put(ins[-1].reshape(m, 1, order="F"), dt)
    by, py, _ = dev.put(np.full((m, n), np.nan, np.float32), dt)
    bp, pp = None, None
    if want_pre:
        bp, pp, _ = dev.put(np.full((m, n), np.nan, np.float32), dt)
    dev.lib.call("ginn_hip_affine_fwd", dev.ctx, dt, act, m, n, pairs,
                 (ctypes.c_void_p * pairs)(*Wp), (ctypes.c_void_p * pairs)(*Xp),
                 (ctypes.c_int * pairs)(*ks), ctypes.c_void_p(pb),
                 ctypes.c_void_p(pp) if want_pre else None, ctypes.c_void_p(py))
    dev.sync()
    Y = dev.get(by, (m, n))
    pre = dev.get(bp, (m, n)) if want_pre else None
    return Y, pre


@pytest.mark.parametrize("dt", DTYPES)
def test_reference_affine_goldens(dev, golden, dt):
    from gpu_util import round_to
    eps = {capi.F32: 1e-6, capi.F16: 2e-3, capi.BF16: 2e-2}[dt]  # Real / Half eps of the reference; bf16 is ours
    g = golden["affine"]
    W, V, b = (farr(g[k], np.float32) for k in ("W", "V", "b"))
    for act, key in ((N.IDENTITY, "WVb"), (N.SIGMOID, "sigmoid_WVb"), (N.SOFTMAX, "softmax_WVb")):
        Y, _ = affine_fwd(dev, dt, act, [W, V, b], want_pre=N.backward_requires_input(act))
        np.testing.assert_allclose(Y, farr(g[key], np.float32), rtol=eps)
    g = golden["affine_broadcast"]
    Y, _ = affine_fwd(dev, dt, N.IDENTITY, [farr(g["W"], np.float32), farr(g["V"], np.float32), farr(g["b"], np.float32)], False)
    np.testing.assert_allclose(Y, farr(g["WVb"], np.float32), rtol=eps)
    g = golden["affine_high_rank"]
    Y, _ = affine_fwd(dev, dt, N.IDENTITY, [farr(g["W"], np.float32), farr(g["V"], np.float32), farr(g["b"], np.float32)], False)
    np.testing.assert_allclose(Y.reshape((2, 2, 2), order="F"), farr(g["WVb"], np.float32), rtol=eps)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("shape", [(5, 3, 7, 0), (64, 33, 48, 0), (130, 70, 96, 40), (512, 64, 784, 0),
                                   (10, 64, 512, 0), (256, 256, 128, 64), (512, 2048, 256, 0),
                                   (384, 128, 2048, 0), (3072, 4096, 256, 0), (1024, 1, 384, 0),
                                   (2048, 8, 640, 64), (256, 64, 128, 0), (64, 256, 256, 64), (512, 40, 192, 0),
                                   (1024, 512, 256, 64),
                                   # tall A, at most 16 columns, long K: one launch of 16-row strips, fused epilogue
                                   (2048, 5, 1024, 1040), (4104, 16, 1040, 0),
                                   # odd leading dimensions, large: the products run on padded copies
                                   (1001, 1003, 1005, 0), (1501, 1503, 1505, 515)])
def test_affine_forward(dev, dt, act, shape):
    """m, n, k, k2 (k2 > 0 adds a second (W, X) pair).  For the 16-bit types the
    aligned shapes take the tuned kernels with their fused epilogues: 128 x 128
    tiles (256 x 256 x 128 + 64, 512 x 2048 x 256, split-K for 384 x 128 x 2048)
    and 256 x 256 tiles (3072 x 4096 x 256).  Tall A with few columns
    (1024 x 1 x 384, 2048 x 8 x 640 + 64) takes the streaming kernel."""
    from gpu_util import TOL, round_to
    m, n, k, k2 = shape
    rng = np.random.default_rng(m + n + k + act)
    ins = [round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt), round_to(rng.standard_normal((k, n)), dt)]
    if k2:
        ins += [round_to(rng.standard_normal((m, k2)) / np.sqrt(k2), dt), round_to(rng.standard_normal((k2, n)), dt)]
    ins.append(round_to(rng.standard_normal((m,)), dt))
    need_pre = N.backward_requires_input(act)
    Y, pre = affine_fwd(dev, dt, act, ins, want_pre=need_pre)
    want, want_pre = N.affine_forward(act, [x.astype(np.float64) for x in ins])
    # Two pairs round the running sum to the storage type once in between.
    tol = TOL[dt] * (2 if k2 else 1)
    assert rel_fro(Y, want) <= tol
    if need_pre:
        assert rel_fro(pre, want_pre) <= tol


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("act", [N.IDENTITY, N.GELU, N.TANH])
def test_affine_forward_two_pairs_large(dev, dt, act):
    """Two (W, X) pairs on a shape of the 256 x 256 kernel (4096 x 4096, k = 256
    and 64): its second product accumulates into what the first left (the
    pre-activation buffer when one is kept, Y otherwise) -- the epilogue that
    reads the old values in batches -- and applies bias and activation."""
    from gpu_util import TOL, round_to
    m, n, k, k2 = 4096, 4096, 256, 64
    rng = np.random.default_rng(act + dt)
    ins = [round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt), round_to(rng.standard_normal((k, n)), dt),
           round_to(rng.standard_normal((m, k2)) / np.sqrt(k2), dt), round_to(rng.standard_normal((k2, n)), dt),
           round_to(rng.standard_normal((m,)), dt)]
    need_pre = N.backward_requires_input(act)
    Y, pre = affine_fwd(dev, dt, act, ins, want_pre=need_pre)
    want, want_pre = N.affine_forward(act, [x.astype(np.float64) for x in ins])
    assert rel_fro(Y, want) <= TOL[dt] * 2
    if need_pre:
        assert rel_fro(pre, want_pre) <= TOL[dt] * 2


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("act", ACTS)
@pytest.mark.parametrize("m,n", [(3, 5), (64, 64), (300, 77), (10, 64), (1024, 512)])
@pytest.mark.parametrize("with_bias", [True, False])
def test_affine_backward_pre(dev, dt, act, m, n, with_bias):
    """dpre = act'(.) * dY and dbias += rowsum(dpre) (ginn/node/affine.h:80-93,107)."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(m * n + act)
    pre = round_to(rng.standard_normal((m, n)), dt)
    Y = round_to(N.nonlin_forward(act, pre.astype(np.float64)), dt)
    dY = round_to(rng.standard_normal((m, n)), dt)
    dbias0 = round_to(rng.standard_normal((m,)), dt)
    b_dy, p_dy, _ = dev.put(dY, dt)
    b_y, p_y, _ = dev.put(Y, dt)
    b_pre, p_pre, _ = dev.put(pre, dt)
    b_dp, p_dp, _ = dev.put(np.full((m, n), np.nan, np.float32), dt)
    b_db, p_db, _ = dev.put(dbias0.reshape(m, 1), dt)
    needs_x = N.backward_requires_input(act) and act != N.SOFTMAX
    dev.lib.call("ginn_hip_affine_bwd_pre", dev.ctx, dt, act, m, n, ctypes.c_void_p(p_dy),
                 ctypes.c_void_p(p_y), ctypes.c_void_p(p_pre) if needs_x else None,
                 ctypes.c_void_p(p_dp) if act != N.IDENTITY else None,
                 ctypes.c_void_p(p_db) if with_bias else None)
    dev.sync()
    want_dpre = N.nonlin_backward(act, dY.astype(np.float64), pre.astype(np.float64), Y.astype(np.float64))
    if act != N.IDENTITY:
        got_dpre = dev.get(b_dp, (m, n))
        assert rel_fro(got_dpre, want_dpre) <= TOL[dt]
        summed = round_to(got_dpre, dt).astype(np.float64)  # the row sum is taken over the stored values
    else:
        summed = dY.astype(np.float64)
    got_db = dev.get(b_db, (m,))
    if with_bias:
        want_db = dbias0 + summed.sum(axis=1)
        # the accumulated bias gradient is rounded once more to the storage type
        assert rel_fro(got_db, want_db) <= TOL[dt] * 2
    else:
        np.testing.assert_array_equal(got_db, dbias0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("act", [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.GELU, N.GELU2, N.SOFTMAX, N.LOG, N.SQRT])
@pytest.mark.parametrize("rows,cols", [(2, 3), (33, 17), (512, 96), (1, 7)])
def test_nonlin_forward_backward(dev, golden, dt, act, rows, cols):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows * cols + act)
    x = rng.standard_normal((rows, cols))
    if act in (N.LOG, N.SQRT):
        x = np.abs(x) + 0.5
    x = round_to(x, dt)
    b_x, p_x, _ = dev.put(x, dt)
    b_y, p_y, _ = dev.put(np.full((rows, cols), np.nan, np.float32), dt)
    dev.lib.call("ginn_hip_nonlin_fwd", dev.ctx, dt, act, rows, cols, ctypes.c_void_p(p_x), ctypes.c_void_p(p_y))
    dev.sync()
    y = dev.get(b_y, (rows, cols))
    want = N.nonlin_forward(act, x.astype(np.float64))
    assert rel_fro(y, want) <= TOL[dt]
    dy = round_to(rng.standard_normal((rows, cols)), dt)
    dx0 = round_to(rng.standard_normal((rows, cols)), dt)
    b_dy, p_dy, _ = dev.put(dy, dt)
    for accumulate in (0, 1):
        b_dx, p_dx, _ = dev.put(dx0, dt)
        dev.lib.call("ginn_hip_nonlin_bwd", dev.ctx, dt, act, rows, cols, ctypes.c_void_p(p_dy),
                     ctypes.c_void_p(p_x), ctypes.c_void_p(p_y), ctypes.c_void_p(p_dx), accumulate)
        dev.sync()
        got = dev.get(b_dx, (rows, cols))
        want_dx = N.nonlin_backward(act, dy.astype(np.float64), x.astype(np.float64), y.astype(np.float64))
        if accumulate:
            want_dx = want_dx + dx0
        assert rel_fro(got, want_dx) <= TOL[dt] * 2


@pytest.mark.parametrize("dt", DTYPES)
def test_nonlin_reference_goldens(dev, golden, dt):
    # test/nodes.cu.cpp:689-753 incl. the saturation cases
    eps = {capi.F32: 1e-6, capi.F16: 1e-3, capi.BF16: 1e-2}[dt]
    g = golden["nonlin"]
    W = farr(g["W"], np.float32)

    def fwd(act, x):
        b_x, p_x, _ = dev.put(x, dt)
        b_y, p_y, _ = dev.put(np.full(x.shape, np.nan, np.float32), dt)
        dev.lib.call("ginn_hip_nonlin_fwd", dev.ctx, dt, act, x.shape[0], x.shape[1], ctypes.c_void_p(p_x), ctypes.c_void_p(p_y))
        dev.sync()
        return dev.get(b_y, x.shape)

    for act, key in ((N.TANH, "tanh"), (N.RELU, "relu"), (N.SIGMOID, "sigmoid"), (N.SOFTMAX, "softmax")):
        np.testing.assert_allclose(fwd(act, W), farr(g[key], np.float32), rtol=max(eps, 1e-6), atol=1e-7 if dt == capi.F32 else 2e-4)
    e = golden["nonlin_extreme"]
    x = farr(e["x"], np.float32)
    x2 = farr(e["x2"], np.float32)
    np.testing.assert_allclose(fwd(N.TANH, x), farr(e["tanh_x"], np.float32), rtol=eps)
    np.testing.assert_allclose(fwd(N.SIGMOID, x), farr(e["sigmoid_x"], np.float32), rtol=eps, atol=1e-30)
    np.testing.assert_allclose(fwd(N.SOFTMAX, x), farr(e["softmax_x"], np.float32), rtol=eps, atol=1e-30)
    np.testing.assert_allclose(fwd(N.SOFTMAX, x.reshape((1, 2), order="F")), farr(e["softmax_x_as_row"], np.float32), rtol=eps)
    np.testing.assert_allclose(fwd(N.SOFTMAX, x2), farr(e["softmax_x2"], np.float32), rtol=eps, atol=1e-30)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(1, 1), (7, 5), (512, 300), (768, 64), (100, 4096)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_col_dot_and_degenerate_batched_gemm(dev, dt, rows, cols, beta):
    """The m = n = 1 batched product of SoftmaxOp::backward / LayerNorm backward
    (ginn/nonlin.h:177-184, ginn/node/layernorm.h:60-64): both the dedicated
    entry point and the batched GEMM routed to it."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows + cols)
    x = round_to(rng.standard_normal((rows, cols)), dt)
    y = round_to(rng.standard_normal((rows, cols)), dt)
    out0 = round_to(rng.standard_normal((cols,)), dt)
    want = (x.astype(np.float64) * y).sum(axis=0) + beta * out0
    b_x, p_x, _ = dev.put(x, dt)
    b_y, p_y, _ = dev.put(y, dt)
    b_o, p_o, _ = dev.put(out0.reshape(cols, 1), dt)
    dev.lib.call("ginn_hip_col_dot_batched", dev.ctx, dt, rows, cols, ctypes.c_void_p(p_x), ctypes.c_void_p(p_y), beta, ctypes.c_void_p(p_o))
    dev.sync()
    assert rel_fro(dev.get(b_o, (cols,)), want) <= TOL[dt]
    # Same through gpu_batched_prod's argument mapping: y_[1, rows, cols] * dy_[rows, 1, cols].
    b_o2, p_o2, _ = dev.put(out0.reshape(cols, 1), dt)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, 0, 0, 1, 1, rows,
                 ctypes.c_void_p(p_x), 1, rows, ctypes.c_void_p(p_y), max(rows, 1), rows, beta,
                 ctypes.c_void_p(p_o2), 1, 1, cols)
    dev.sync()
    assert rel_fro(dev.get(b_o2, (cols,)), want) <= TOL[dt]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a", [0, 1])
@pytest.mark.parametrize("ns", [[1, 1, 1], [3, 1, 7, 2], [64] * 5, [1] * 200, [5, 0, 9]])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_grouped_gemm(dev, dt, op_a, ns, beta):
    """Products sharing the left operand (what Autobatch forms by concatenating
    right-hand sides, ginn/autobatch.h:149-183) == the per-group products."""
    from gpu_util import TOL, round_to
    m, k = 96, 72
    rng = np.random.default_rng(len(ns) + sum(ns))
    A = round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt)
    As = np.asfortranarray(A.T) if op_a else A
    ba, pa, lda = dev.put(As, dt)
    Bs = [round_to(rng.standard_normal((k, n)), dt) for n in ns]
    Cs = [round_to(rng.standard_normal((m, n)), dt) for n in ns]
    keep, pB, pC, ldb, ldc = [], [], [], [], []
    for Bm, Cm in zip(Bs, Cs):
        bb, pb, lb = dev.put(Bm, dt, pad_rows=8 if Bm.shape[1] > 1 else 0)
        bc, pc, lc = dev.put(Cm, dt)
        keep += [bb, bc]
        pB.append(pb); pC.append(pc); ldb.append(lb); ldc.append(lc)
    g = len(ns)
    dev.lib.call("ginn_hip_gemm_grouped", dev.ctx, dt, op_a, m, k, ctypes.c_void_p(pa), lda, g,
                 (ctypes.c_void_p * g)(*pB), (ctypes.c_int * g)(*ns), (ctypes.c_int * g)(*ldb), beta,
                 (ctypes.c_void_p * g)(*pC), (ctypes.c_int * g)(*ldc))
    dev.sync()
    for i, n in enumerate(ns):
        if n == 0:
            continue
        want = A.astype(np.float64) @ Bs[i] + beta * Cs[i]
        got = dev.get(keep[2 * i + 1], (m, n), ldc[i])
        assert rel_fro(got, want) <= TOL[dt], (i, n)


def _scatter_columns(dev, M, dt, rng, misalign=False):
    """Puts every column of M into one device buffer in shuffled order with
    gaps between them; returns (buffer, bytes per element, element offset of
    every column, device table of the column addresses)."""
    rows, cols = M.shape
    stride = (rows + 7) // 8 * 8 + 8
    order = rng.permutation(cols)
    shift = 1 if misalign else 0
    big = np.full((stride, cols + 1), np.nan, np.float32, order="F")
    offs = np.zeros(cols, np.int64)
    for slot, c in enumerate(order):
        big[shift:shift + rows, slot] = M[:, c]
        offs[c] = slot * stride + shift
    buf, ptr, ld = dev.put(big, dt)
    assert ld == stride
    es = 4 if dt == capi.F32 else 2
    table = np.array([ptr + es * int(o) for o in offs], np.uint64).view(np.int64)
    tbuf = dev.torch.from_numpy(table).to(device="cuda")
    return (buf, tbuf), big.shape, offs, tbuf.data_ptr()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,k,n", [(96, 72, 40), (64, 64, 64), (130, 33, 7), (1024, 384, 200), (8, 8, 1),
                                   (1024, 384, 100)])  # fp32: the scattered dX on 16 x 16 tiles
@pytest.mark.parametrize("misalign", [False, True])
def test_gathered_gemm(dev, dt, m, k, n, misalign):
    """The three products of a merged Autobatch group on operands that stay
    where they are (ginn/autobatch.h:149-183 without RowwiseCat's copy):
    Y = W [x_0 x_1 ...] with gathered columns, dW += dY [x_0 x_1 ...]^T summing
    over the gathered columns, dx_i += W^T dY_i into scattered columns."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(m * 7 + k * 3 + n + misalign)
    W = round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt)
    X = round_to(rng.standard_normal((k, n)), dt)
    dY = round_to(rng.standard_normal((m, n)) / np.sqrt(m), dt)
    dW0 = round_to(rng.standard_normal((m, k)), dt)
    dX0 = round_to(rng.standard_normal((k, n)), dt)
    bw, pw, ldw = dev.put(W, dt)
    keep_x, shape_x, offs_x, table_x = _scatter_columns(dev, X, dt, rng, misalign)
    aligned = 0 if misalign else 1
    vp = ctypes.c_void_p

    # forward, beta = 0
    by, py, ldy = dev.put(np.full((m, n), np.nan, np.float32), dt)
    dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, dt, 0, 0, m, n, k, vp(pw), ldw, None, 0, vp(table_x), 0.0,
                 vp(py), ldy, None, aligned)
    dev.sync()
    assert rel_fro(dev.get(by, (m, n), ldy), W.astype(np.float64) @ X) <= TOL[dt]

    # gradient of the shared left operand, beta = 1: sums over the gathered columns
    bdy, pdy, lddy = dev.put(dY, dt)
    bdw, pdw, lddw = dev.put(dW0, dt)
    dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, dt, 0, 1, m, k, n, vp(pdy), lddy, None, 0, vp(table_x), 1.0,
                 vp(pdw), lddw, None, aligned)
    dev.sync()
    assert rel_fro(dev.get(bdw, (m, k), lddw), dY.astype(np.float64) @ X.T + dW0) <= TOL[dt]

    # gradients of the right operands, beta = 1, into scattered columns
    keep_g, shape_g, offs_g, table_g = _scatter_columns(dev, dX0, dt, rng, misalign)
    dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, dt, 1, 0, k, n, m, vp(pw), ldw, vp(pdy), lddy, None, 1.0,
                 None, 0, vp(table_g), aligned)
    dev.sync()
    flat = dev.get(keep_g[0], shape_g).reshape(-1, order="F")
    got = np.stack([flat[o:o + k] for o in offs_g], axis=1)
    assert rel_fro(got, W.astype(np.float64).T @ dY + dX0) <= TOL[dt]
    # nothing outside the columns was written
    mask = np.ones(flat.size, bool)
    for o in offs_g:
        mask[o:o + k] = False
    assert np.isnan(flat[mask]).all()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,n,k", [(96, 72, 40), (64, 64, 300), (130, 33, 7), (1024, 384, 1500), (8, 12, 1), (5, 3, 0),
                                   (96, 72, 600), (50, 19, 1024)])  # fp32: both tables on 16 x 16 tiles
@pytest.mark.parametrize("misalign", [False, True])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_outer_sum_of_scattered_columns(dev, dt, m, n, k, misalign, beta):
    """ginn_hip_gemm_outer_sum: dW = sum_j dy_j x_j^T + beta dW over column
    pairs that lie anywhere -- what the accumulating dA += dY B^T of every
    product sharing A (ginn/node/prod.h:57-63) adds up to."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(m * 11 + n * 5 + k + misalign)
    dY = round_to(rng.standard_normal((m, max(k, 1))) / np.sqrt(max(k, 1)), dt)[:, :k]
    X = round_to(rng.standard_normal((n, max(k, 1))), dt)[:, :k]
    dW0 = round_to(rng.standard_normal((m, n)), dt)
    vp = ctypes.c_void_p
    table_a = table_b = None
    if k > 0:
        keep_a, _, _, table_a = _scatter_columns(dev, dY, dt, rng, misalign)
        keep_b, _, _, table_b = _scatter_columns(dev, X, dt, rng, misalign)
    start = dW0 if beta else np.full((m, n), np.nan, np.float32)
    bw, pw, ldw = dev.put(start, dt)
    dev.lib.call("ginn_hip_gemm_outer_sum", dev.ctx, dt, m, n, k, vp(table_a) if k else None,
                 vp(table_b) if k else None, beta, vp(pw), ldw, 0 if misalign else 1)
    dev.sync()
    want = dY.astype(np.float64) @ X.astype(np.float64).T + (dW0 if beta else 0)
    got = dev.get(bw, (m, n), ldw)
    if k == 0 and not beta:
        assert (got == 0).all()
    else:
        assert rel_fro(got, want) <= TOL[dt]


def test_outer_sum_argument_checks(dev):
    vp = ctypes.c_void_p
    b, p, ld = dev.put(np.zeros((8, 8), np.float32), capi.F32)
    with pytest.raises(capi.GinnHipError, match="NULL table"):
        dev.lib.call("ginn_hip_gemm_outer_sum", dev.ctx, capi.F32, 8, 8, 4, None, vp(p), 0.0, vp(p), 8, 1)
    with pytest.raises(capi.GinnHipError, match="ldc"):
        dev.lib.call("ginn_hip_gemm_outer_sum", dev.ctx, capi.F32, 8, 8, 4, vp(p), vp(p), 0.0, vp(p), 4, 1)
    with pytest.raises(capi.GinnHipError, match="C is NULL"):
        dev.lib.call("ginn_hip_gemm_outer_sum", dev.ctx, capi.F32, 8, 8, 4, vp(p), vp(p), 0.0, None, 8, 1)


def test_gathered_gemm_argument_checks(dev):
    vp = ctypes.c_void_p
    b, p, ld = dev.put(np.zeros((8, 8), np.float32), capi.F32)
    with pytest.raises(capi.GinnHipError, match="lda"):
        dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, capi.F32, 0, 0, 8, 8, 8, vp(p), 4, None, 0, vp(p), 0.0,
                     vp(p), 8, None, 1)
    with pytest.raises(capi.GinnHipError, match="C is NULL"):
        dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, capi.F32, 0, 0, 8, 8, 8, vp(p), 8, None, 0, vp(p), 0.0,
                     None, 8, None, 1)
    # without tables: an ordinary product
    A = np.arange(64, dtype=np.float32).reshape(8, 8, order="F") / 64
    ba, pa, _ = dev.put(A, capi.F32)
    bc, pc, _ = dev.put(np.zeros((8, 8), np.float32), capi.F32)
    dev.lib.call("ginn_hip_gemm_gathered", dev.ctx, capi.F32, 0, 0, 8, 8, 8, vp(pa), 8, vp(pa), 8, None, 0.0,
                 vp(pc), 8, None, 1)
    dev.sync()
    np.testing.assert_allclose(dev.get(bc, (8, 8)), A.astype(np.float64) @ A, rtol=1e-5)


# Column lengths on both sides of every variant of the column softmax: the
# three-pass kernels (unaligned rows, or more than 8192 rows) and the
# column-in-registers kernels with 1, 2, 4, 8 and 16 vectors per lane, with
# ragged last vectors and column counts that do not fill a wave's group.
SOFTMAX_SHAPES = [(8, 9), (504, 7), (512, 13), (520, 5), (1000, 6), (2048, 3), (2056, 2), (4104, 5),
                  (8192, 3), (8200, 2), (1001, 4)]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", SOFTMAX_SHAPES)
def test_softmax_column_variants(dev, dt, rows, cols):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows * 31 + cols)
    x = round_to(rng.standard_normal((rows, cols)) * 3, dt)
    b_x, p_x, _ = dev.put(x, dt)
    b_y, p_y, _ = dev.put(np.full((rows, cols), np.nan, np.float32), dt)
    dev.lib.call("ginn_hip_nonlin_fwd", dev.ctx, dt, N.SOFTMAX, rows, cols, ctypes.c_void_p(p_x), ctypes.c_void_p(p_y))
    dev.sync()
    y = dev.get(b_y, (rows, cols))
    want = N.nonlin_forward(N.SOFTMAX, x.astype(np.float64))
    assert rel_fro(y, want) <= TOL[dt]
    np.testing.assert_allclose(y.sum(axis=0), 1.0, atol={capi.F32: 1e-5}.get(dt, 2e-2))
    # in place (ginn/node/inplace.h): same bits
    dev.lib.call("ginn_hip_nonlin_fwd", dev.ctx, dt, N.SOFTMAX, rows, cols, ctypes.c_void_p(p_x), ctypes.c_void_p(p_x))
    dev.sync()
    np.testing.assert_array_equal(dev.get(b_x, (rows, cols)), y)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", SOFTMAX_SHAPES + [(10, 64), (3, 1)])
def test_pick_neg_log_softmax(dev, dt, rows, cols):
    """ginn_hip_pick_nls_fwd / _bwd against ginn/node/pick.h:178-236: the loss is
    -log of the STORED softmax value, the gradient softmax - onehot scaled by
    the incoming gradient of each column, accumulated."""
    from gpu_util import TOL, round_to
    torch = dev.torch
    rng = np.random.default_rng(rows * 17 + cols)
    x = round_to(rng.standard_normal((rows, cols)) * 2, dt)
    labels = rng.integers(0, rows, size=cols).astype(np.int32)
    labels[0], labels[-1] = rows - 1, 0
    b_x, p_x, _ = dev.put(x, dt)
    b_s, p_s, _ = dev.put(np.full((rows, cols), np.nan, np.float32), dt)
    b_o, p_o, _ = dev.put(np.full((1, cols), np.nan, np.float32), dt)
    idx = torch.from_numpy(labels).cuda()
    dev.lib.call("ginn_hip_pick_nls_fwd", dev.ctx, dt, rows, cols, ctypes.c_void_p(p_x),
                 ctypes.c_void_p(idx.data_ptr()), ctypes.c_void_p(p_s), ctypes.c_void_p(p_o))
    dev.sync()
    sm = dev.get(b_s, (rows, cols))
    nll = dev.get(b_o, (1, cols)).ravel()
    want_nll, want_sm = N.pick_neg_log_softmax(x.astype(np.float64), labels)
    assert rel_fro(sm, want_sm) <= TOL[dt]
    # the loss comes from the stored (rounded) probability
    np.testing.assert_allclose(nll, -np.log(sm[labels, np.arange(cols)].astype(np.float64)),
                               rtol={capi.F32: 1e-5}.get(dt, 1e-2), atol={capi.F32: 1e-6}.get(dt, 1e-2))
    assert rel_fro(nll, want_nll) <= TOL[dt] * 2

    dout = round_to(rng.standard_normal((1, cols)), dt)
    dx0 = round_to(rng.standard_normal((rows, cols)), dt)
    b_d, p_d, _ = dev.put(dout, dt)
    b_dx, p_dx, _ = dev.put(dx0, dt)
    dev.lib.call("ginn_hip_pick_nls_bwd", dev.ctx, dt, rows, cols, ctypes.c_void_p(p_s),
                 ctypes.c_void_p(idx.data_ptr()), ctypes.c_void_p(p_d), ctypes.c_void_p(p_dx))
    dev.sync()
    onehot = np.zeros((rows, cols))
    onehot[labels, np.arange(cols)] = 1.0
    want_dx = dx0 + (sm.astype(np.float64) - onehot) * dout.astype(np.float64)
    assert rel_fro(dev.get(b_dx, (rows, cols)), want_dx) <= TOL[dt] * 2

    # The pair that keeps two numbers per column instead of the softmax matrix: the same loss bits; the
    # gradient, adding and assigning, as from the stored softmax (for half storage a few results per
    # million may differ in the last bit: the product with 1 / sum is rounded to half by one instruction
    # in one kernel and by two in the other).
    b_t = torch.full((2 * cols,), float("nan"), device="cuda", dtype=torch.float32)
    b_o2, p_o2, _ = dev.put(np.full((1, cols), np.nan, np.float32), dt)
    dev.lib.call("ginn_hip_pick_nls_fwd_stats", dev.ctx, dt, rows, cols, ctypes.c_void_p(p_x),
                 ctypes.c_void_p(idx.data_ptr()), ctypes.c_void_p(b_t.data_ptr()), ctypes.c_void_p(p_o2))
    for accumulate in (1, 0):
        b_dx2, p_dx2, _ = dev.put(dx0, dt)
        dev.lib.call("ginn_hip_pick_nls_bwd_stats", dev.ctx, dt, rows, cols, ctypes.c_void_p(p_x),
                     ctypes.c_void_p(b_t.data_ptr()), ctypes.c_void_p(idx.data_ptr()), ctypes.c_void_p(p_d),
                     ctypes.c_void_p(p_dx2), accumulate)
        b_ref, p_ref, _ = dev.put(dx0, dt)
        dev.lib.call("ginn_hip_pick_nls_bwd" if accumulate else "ginn_hip_pick_nls_bwd_assign", dev.ctx, dt, rows,
                     cols, ctypes.c_void_p(p_s), ctypes.c_void_p(idx.data_ptr()), ctypes.c_void_p(p_d),
                     ctypes.c_void_p(p_ref))
        dev.sync()
        got, ref = dev.get(b_dx2, (rows, cols)), dev.get(b_ref, (rows, cols))
        if dt == capi.F16:
            differ = got != ref
            assert differ.mean() <= 1e-4 or differ.sum() <= 1
            ulp = np.spacing(np.maximum(np.abs(got[differ]), np.abs(ref[differ])).astype(np.float16)).astype(np.float32)
            assert np.all(np.abs(got[differ] - ref[differ]) <= ulp)
        else:
            np.testing.assert_array_equal(got, ref)
        if not accumulate:
            assert rel_fro(got, (sm.astype(np.float64) - onehot) * dout.astype(np.float64)) <= TOL[dt] * 2
    np.testing.assert_array_equal(dev.get(b_o2, (1, cols)).ravel(), nll)
    stats = b_t.cpu().numpy().reshape(cols, 2)
    np.testing.assert_allclose(stats[:, 0], x.max(axis=0), rtol=0, atol=0)
    np.testing.assert_allclose(1.0 / stats[:, 1], np.exp(x.astype(np.float64) - x.max(axis=0)).sum(axis=0),
                               rtol={capi.F32: 1e-5}.get(dt, 5e-3))
