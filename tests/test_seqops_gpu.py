"""Transformer-block companions through the C ABI (layer normalisation, the
gamma / beta affine, axis permutation, masked fill, causal mask) and the GPT
decoder layer built with the C++ host layer, against the numpy oracle."""
import ctypes
import itertools
from ctypes import c_void_p
from pathlib import Path

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi
from oracle import nodes as N

pytestmark = pytest.mark.gpu

DTYPES = [capi.F32, capi.F16, capi.BF16]
SHIM = capi.LIB_PATH.parent / "libginn_examples.so"
FP = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def dev():
    from gpu_util import Dev
    d = Dev()
    yield d
    d.close()


@pytest.fixture(scope="module")
def shim():
    if not SHIM.exists():
        pytest.fail(f"{SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(SHIM))
    lib.scenario_last_error.restype = ctypes.c_char_p
    return lib


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(768, 64), (5, 3), (1, 4), (64, 1), (100, 33), (1030, 7)])
def test_layernorm(dev, dt, rows, cols):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows + cols)
    x = round_to(rng.standard_normal((rows, cols)) * 2 + 0.5, dt)
    dy = round_to(rng.standard_normal((rows, cols)), dt)
    bx, px, _ = dev.put(x, dt)
    by, py, _ = dev.put(np.zeros_like(x), dt)
    bdy, pdy, _ = dev.put(dy, dt)
    base = round_to(rng.standard_normal((rows, cols)), dt)
    bdx, pdx, _ = dev.put(base, dt)
    std = dev.torch.zeros(cols, dtype=dev.torch.float32, device="cuda")
    eps = 1e-8
    dev.lib.call("ginn_hip_layernorm_fwd", dev.ctx, dt, rows, cols, c_void_p(px), eps, c_void_p(py),
                 c_void_p(std.data_ptr()))
    dev.lib.call("ginn_hip_layernorm_bwd", dev.ctx, dt, rows, cols, c_void_p(pdy), c_void_p(py),
                 c_void_p(std.data_ptr()), c_void_p(pdx))
    dev.sync()
    want_y, want_std = N.layernorm_forward(x.astype(np.float64), eps)
    got_y = dev.get(by, (rows, cols))
    if rows > 1:
        assert rel_fro(got_y, want_y) <= TOL[dt]
        np.testing.assert_allclose(std.cpu().numpy(), want_std, rtol=1e-5)
    else:  # a single row: x - mean = 0, std = sqrt(eps)
        assert not got_y.any()
    # backward from the values the device stored (as the node does)
    want_dx = base + N.layernorm_backward(dy.astype(np.float64), got_y.astype(np.float64),
                                          std.cpu().numpy().astype(np.float64))
    assert rel_fro(dev.get(bdx, (rows, cols)), want_dx) <= TOL[dt]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols", [(768, 520), (64, 5), (8, 3), (1536, 33), (2048, 70), (520, 1030), (12, 7),
                                       (2056, 9), (300, 5)])
@pytest.mark.parametrize("accumulate", [0, 1])
def test_layernorm_affine_as_one_pass(dev, dt, rows, cols, accumulate):
    """ginn_hip_layernorm_affine_fwd / _bwd against ginn_hip_layernorm_fwd + ginn_hip_cwise_prod_add_fwd and
    ginn_hip_cwise_prod_add_bwd_assign + ginn_hip_layernorm_bwd(_assign): normalised values, statistics and z
    bit for bit; dx and the gamma / beta gradients (row sums taken in another order of the columns) within fp32
    rounding; and all of it against numpy.  Columns of 1, 2 and 4 vectors per lane, columns that
    are not multiples of 8 (scalar accesses) and ones too long for the registers (the two steps inside)."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows * 7 + cols)
    x = round_to(rng.standard_normal((rows, cols)) * 2 + 0.5, dt)
    gamma = round_to(rng.standard_normal(rows) * 0.3, dt)
    beta = round_to(rng.standard_normal(rows), dt)
    dz = round_to(rng.standard_normal((rows, cols)), dt)
    old_dx = round_to(rng.standard_normal((rows, cols)), dt)
    old_dg = round_to(rng.standard_normal(rows), dt)
    old_db = round_to(rng.standard_normal(rows), dt)
    mb, eps = 1.0, 1e-8
    t = dev.torch
    put = lambda a: dev.put(a, dt)
    (bx, px, _), (bg, pg, _), (bb, pb, _), (bdz, pdz, _) = put(x), put(gamma), put(beta), put(dz)

    def separate():
        (by, py, _), (bz, pz, _), (bda, pda, _) = put(np.zeros_like(x)), put(np.zeros_like(x)), put(np.full_like(x, 3.0))
        (bdx, pdx, _), (bdg, pdg, _), (bdb, pdb, _) = put(old_dx), put(old_dg), put(old_db)
        std = t.zeros(cols, dtype=t.float32, device="cuda")
        dev.lib.call("ginn_hip_layernorm_fwd", dev.ctx, dt, rows, cols, c_void_p(px), eps, c_void_p(py),
                     c_void_p(std.data_ptr()))
        dev.lib.call("ginn_hip_cwise_prod_add_fwd", dev.ctx, dt, rows, cols, c_void_p(py), c_void_p(pg), c_void_p(pb),
                     mb, 1, c_void_p(pz))
        dev.lib.call("ginn_hip_cwise_prod_add_bwd_assign", dev.ctx, dt, rows, cols, c_void_p(pdz), c_void_p(py),
                     c_void_p(pg), mb, 1, c_void_p(pda), c_void_p(pdg), c_void_p(pdb))
        dev.lib.call("ginn_hip_layernorm_bwd" if accumulate else "ginn_hip_layernorm_bwd_assign", dev.ctx, dt, rows,
                     cols, c_void_p(pda), c_void_p(py), c_void_p(std.data_ptr()), c_void_p(pdx))
        dev.sync()
        return [dev.get(b, s) for b, s in ((by, x.shape), (bz, x.shape), (bdx, x.shape), (bdg, (rows,)),
                                           (bdb, (rows,)))] + [std.cpu().numpy()]

    def fused():
        (by, py, _), (bz, pz, _) = put(np.zeros_like(x)), put(np.zeros_like(x))
        (bdx, pdx, _), (bdg, pdg, _), (bdb, pdb, _) = put(old_dx), put(old_dg), put(old_db)
        std = t.zeros(cols, dtype=t.float32, device="cuda")
        dev.lib.call("ginn_hip_layernorm_affine_fwd", dev.ctx, dt, rows, cols, c_void_p(px), eps, c_void_p(pg),
                     c_void_p(pb), mb, c_void_p(py), c_void_p(std.data_ptr()), c_void_p(pz))
        dev.lib.call("ginn_hip_layernorm_affine_bwd", dev.ctx, dt, rows, cols, c_void_p(pdz), c_void_p(py),
                     c_void_p(std.data_ptr()), c_void_p(pg), mb, c_void_p(pdx), accumulate, c_void_p(pdg),
                     c_void_p(pdb))
        dev.sync()
        return [dev.get(b, s) for b, s in ((by, x.shape), (bz, x.shape), (bdx, x.shape), (bdg, (rows,)),
                                           (bdb, (rows,)))] + [std.cpu().numpy()]

    y1, z1, dx1, dg1, db1, std1 = separate()
    y2, z2, dx2, dg2, db2, std2 = fused()
    np.testing.assert_array_equal(y2, y1)
    np.testing.assert_array_equal(std2, std1)
    np.testing.assert_array_equal(z2, z1)
    assert rel_fro(dx2, dx1) <= {capi.F32: 1e-6}.get(dt, TOL[dt] / 8)
    # row sums over `cols` terms in fp32, rounded to the storage type once
    assert rel_fro(dg2, dg1) <= {capi.F32: 2e-6}.get(dt, TOL[dt] / 4)
    assert rel_fro(db2, db1) <= {capi.F32: 2e-6}.get(dt, TOL[dt] / 4)
    # against numpy, from the values the device stored
    y64 = y2.astype(np.float64)
    want_z = y64 * (gamma.astype(np.float64)[:, None] + mb) + beta.astype(np.float64)[:, None]
    assert rel_fro(z2, want_z) <= TOL[dt]
    da = round_to(dz.astype(np.float64) * (gamma.astype(np.float64)[:, None] + mb), dt).astype(np.float64)
    want_dx = (old_dx if accumulate else 0) + N.layernorm_backward(da, y64, std2.astype(np.float64))
    if rows > 1:
        assert rel_fro(dx2, want_dx) <= TOL[dt] * 2
    assert rel_fro(dg2, old_dg + (dz.astype(np.float64) * y64).sum(axis=1)) <= TOL[dt]
    assert rel_fro(db2, old_db + dz.astype(np.float64).sum(axis=1)) <= TOL[dt]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("rows,cols,broadcast", [(768, 40, 1), (5, 3, 1), (5, 3, 0), (300, 257, 1), (1, 9, 1)])
def test_cwise_prod_add(dev, dt, rows, cols, broadcast):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(rows * 3 + cols)
    a = round_to(rng.standard_normal((rows, cols)), dt)
    bshape = (rows,) if broadcast else (rows, cols)
    b = round_to(rng.standard_normal(bshape) * 0.1, dt)
    c = round_to(rng.standard_normal(bshape), dt)
    dy = round_to(rng.standard_normal((rows, cols)), dt)
    bufs = {k: dev.put(v, dt) for k, v in dict(a=a, b=b, c=c, dy=dy).items()}
    by, py, _ = dev.put(np.zeros((rows, cols)), dt)
    bda, pda, _ = dev.put(np.zeros((rows, cols)), dt)
    bdb, pdb, _ = dev.put(np.zeros(bshape), dt)
    bdc, pdc, _ = dev.put(np.zeros(bshape), dt)
    P = lambda k: c_void_p(bufs[k][1])
    dev.lib.call("ginn_hip_cwise_prod_add_fwd", dev.ctx, dt, rows, cols, P("a"), P("b"), P("c"), 1.0, broadcast,
                 c_void_p(py))
    dev.lib.call("ginn_hip_cwise_prod_add_bwd", dev.ctx, dt, rows, cols, P("dy"), P("a"), P("b"), 1.0, broadcast,
                 c_void_p(pda), c_void_p(pdb), c_void_p(pdc))
    # a second call accumulates; only db this time
    dev.lib.call("ginn_hip_cwise_prod_add_bwd", dev.ctx, dt, rows, cols, P("dy"), P("a"), P("b"), 1.0, broadcast,
                 None, c_void_p(pdb), None)
    dev.sync()
    a64, b64, c64, dy64 = (v.astype(np.float64) for v in (a, b, c, dy))
    assert rel_fro(dev.get(by, (rows, cols)), N.cwise_prod_add_forward(a64, b64, c64, 1.0)) <= TOL[dt]
    da, db, dc = N.cwise_prod_add_backward(dy64, a64, b64, 1.0)
    assert rel_fro(dev.get(bda, (rows, cols)), da) <= TOL[dt]
    # db was accumulated twice, rounding to the storage type in between
    assert rel_fro(dev.get(bdb, bshape), 2 * db) <= 2 * TOL[dt]
    assert rel_fro(dev.get(bdc, bshape), dc) <= TOL[dt]


PERM_CASES = [((4, 3), (1, 0)), ((64, 12, 8, 16), (3, 0, 2, 1)), ((64, 12, 8, 16), (0, 3, 2, 1)),
              ((64, 16, 8, 12), (0, 3, 2, 1)), ((5, 6, 7), (2, 0, 1)), ((5, 6, 7), (1, 2, 0)), ((33, 70), (1, 0)),
              ((7,), (0,)), ((3, 1, 40, 2), (2, 3, 0, 1)), ((2, 3, 4, 5, 6), (4, 2, 0, 3, 1)),
              ((40, 3, 50), (2, 1, 0)), ((1, 9), (1, 0)),
              # extents that are multiples of 4: 64 x 64 tiles for the 16-bit types (whole and ragged tiles)
              ((512, 64, 12), (1, 0, 2)), ((68, 132), (1, 0)), ((128, 5, 72), (2, 1, 0)), ((64, 3, 4, 200), (3, 1, 0, 2))]


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("shape,perm", PERM_CASES)
def test_permute(dev, dt, shape, perm):
    from gpu_util import round_to
    rng = np.random.default_rng(len(shape))
    x = round_to(rng.standard_normal(shape), dt)
    want = N.permute(x, perm)
    bx, px, _ = dev.put(x.reshape(-1, order="F"), dt)
    bo, po, _ = dev.put(np.zeros(x.size), dt)
    rank = len(shape)
    dims = (ctypes.c_longlong * rank)(*shape)
    pm = (ctypes.c_int * rank)(*perm)
    dev.lib.call("ginn_hip_permute", dev.ctx, dt, rank, dims, pm, c_void_p(px), c_void_p(po), 0)
    dev.sync()
    got = dev.get(bo, (x.size,)).reshape(want.shape, order="F")
    np.testing.assert_array_equal(got, want)  # pure data movement: bit exact
    # backward: accumulate the inverse permutation of the result onto x -> 2 x
    inv = (ctypes.c_int * rank)(*np.argsort(perm).tolist())
    odims = (ctypes.c_longlong * rank)(*want.shape)
    dev.lib.call("ginn_hip_permute", dev.ctx, dt, rank, odims, inv, c_void_p(po), c_void_p(px), 1)
    dev.sync()
    np.testing.assert_array_equal(dev.get(bx, (x.size,)).reshape(shape, order="F"), round_to(2 * x, dt))


def test_permute_rejects_bad_arguments(dev):
    buf = dev.torch.zeros(16, device="cuda")
    dims = (ctypes.c_longlong * 2)(4, 4)
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_permute", dev.ctx, capi.F32, 2, dims, (ctypes.c_int * 2)(0, 0),
                     c_void_p(buf.data_ptr()), c_void_p(buf.data_ptr() + 64), 0)
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_permute", dev.ctx, capi.F32, 9, dims, (ctypes.c_int * 2)(0, 1),
                     c_void_p(buf.data_ptr()), c_void_p(buf.data_ptr()), 0)
    with pytest.raises(capi.GinnHipError):  # in place
        dev.lib.call("ginn_hip_permute", dev.ctx, capi.F32, 2, dims, (ctypes.c_int * 2)(1, 0),
                     c_void_p(buf.data_ptr()), c_void_p(buf.data_ptr()), 0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n,batch", [(4, 3), (33, 5), (1, 1)])
def test_upper_tri_and_mask_fill(dev, dt, n, batch):
    from gpu_util import round_to
    rng = np.random.default_rng(n)
    bm, pm, _ = dev.put(np.zeros((n, n)), dt)
    dev.lib.call("ginn_hip_upper_tri", dev.ctx, dt, n, c_void_p(pm))
    x = round_to(rng.standard_normal((n, n, batch)), dt)
    bx, px, _ = dev.put(x.reshape(-1, order="F"), dt)
    dev.lib.call("ginn_hip_mask_fill", dev.ctx, dt, n * n, batch, c_void_p(pm), float("-inf"), c_void_p(px))
    dev.sync()
    mask = dev.get(bm, (n, n))
    np.testing.assert_array_equal(mask, N.upper_tri(n))
    got = dev.get(bx, (x.size,)).reshape(x.shape, order="F")
    want = np.where(N.upper_tri(n)[:, :, None] != 0, x, -np.inf)
    np.testing.assert_array_equal(got, want)


# ---------------------------------------------------------------------------
# scale -> mask -> softmax of attention scores as one launch
# ---------------------------------------------------------------------------

# (T, batch, offset): scores [T x T x batch], causal mask [T x T]; an offset breaks 16-byte alignment.
# 512: one vector per lane, two columns per wave; 1024, 2048: 2 and 4 vectors; 24: a partly filled
# wave; 20 (rows % 8 != 0), 4096 (column too long for the registers) and the offset case take the
# three separate launches inside the entry point.
SCORE_CASES = [(512, 3, 0), (1024, 1, 0), (2048, 1, 0), (24, 5, 0), (64, 7, 0), (20, 3, 0), (24, 2, 1)]


def _score_inputs(dev, dt, T, batch, offset, seed):
    from gpu_util import round_to
    rng = np.random.default_rng(seed)
    x = round_to(rng.standard_normal((T, T * batch)) * 3, dt)
    dy = round_to(rng.standard_normal((T, T * batch)), dt)
    mask = N.upper_tri(T).astype(np.float32)
    return x, dy, mask


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T,batch,offset", SCORE_CASES + [(4096, 1, 0)])
def test_scaled_masked_softmax_equals_the_three_steps(dev, dt, T, batch, offset):
    """ginn_hip_scaled_masked_softmax_fwd / _bwd against ginn_hip_scale_shift, ginn_hip_mask_fill and
    ginn_hip_nonlin_fwd / _bwd called one after the other (what InPlaceProdScalar, InPlaceMask and
    Softmax do as three nodes): the same bits, in the scores left in place, the softmax and the gradient
    (the gradient in half storage: up to the last bit of a few results per million, see below)."""
    if T == 4096 and dt != capi.BF16:
        pytest.skip("one dtype is enough for the long-column fallback")
    x, dy, mask = _score_inputs(dev, dt, T, batch, offset, seed=T + batch)
    n = x.size
    scale = 1.0 / np.sqrt(64.0)
    flat = lambda a: a.reshape(-1, order="F")
    bm, pm, _ = dev.put(flat(mask), dt)
    # separate steps
    bx1, px1, _ = dev.put(flat(x), dt, offset=offset)
    by1, py1, _ = dev.put(np.zeros(n), dt, offset=offset)
    dev.lib.call("ginn_hip_scale_shift", dev.ctx, dt, n, scale, 0.0, c_void_p(px1), c_void_p(px1), 0)
    dev.lib.call("ginn_hip_mask_fill", dev.ctx, dt, T * T, batch, c_void_p(pm), float("-inf"), c_void_p(px1))
    dev.lib.call("ginn_hip_nonlin_fwd", dev.ctx, dt, capi.ACT_SOFTMAX, T, T * batch, c_void_p(px1), c_void_p(py1))
    bg, pg, _ = dev.put(flat(dy), dt, offset=offset)
    bd1, pd1, _ = dev.put(np.full(n, 7.0), dt, offset=offset)  # overwritten: accumulate = 0
    dev.lib.call("ginn_hip_nonlin_bwd", dev.ctx, dt, capi.ACT_SOFTMAX, T, T * batch, c_void_p(pg), None,
                 c_void_p(py1), c_void_p(pd1), 0)
    dev.lib.call("ginn_hip_mask_fill", dev.ctx, dt, T * T, batch, c_void_p(pm), 0.0, c_void_p(pd1))
    dev.lib.call("ginn_hip_scale_shift", dev.ctx, dt, n, scale, 0.0, c_void_p(pd1), c_void_p(pd1), 0)
    # one launch each way
    bx2, px2, _ = dev.put(flat(x), dt, offset=offset)
    by2, py2, _ = dev.put(np.zeros(n), dt, offset=offset)
    dev.lib.call("ginn_hip_scaled_masked_softmax_fwd", dev.ctx, dt, T, T * batch, c_void_p(px2), scale, c_void_p(pm),
                 T * T, float("-inf"), c_void_p(py2))
    bd2, pd2, _ = dev.put(np.full(n, -3.0), dt, offset=offset)
    dev.lib.call("ginn_hip_scaled_masked_softmax_bwd", dev.ctx, dt, T, T * batch, c_void_p(pg), c_void_p(py2), scale,
                 c_void_p(pm), T * T, c_void_p(pd2))
    dev.sync()
    get = lambda b: dev.get(b, (n,), offset=offset)
    np.testing.assert_array_equal(get(bx2), get(bx1))
    np.testing.assert_array_equal(get(by2), get(by1))
    d1, d2 = get(bd1), get(bd2)
    if dt == capi.F16:
        # A few results per million may differ in the last bit: where a product is converted to half, the
        # compiler emits one instruction that rounds once (v_fma_mixlo_f16) in one kernel and a multiplication
        # in fp32 followed by a conversion, which round twice, in the other.
        differ = d1 != d2
        assert differ.mean() <= 2e-5
        ulp = np.spacing(np.maximum(np.abs(d1[differ]), np.abs(d2[differ])).astype(np.float16)).astype(np.float32)
        assert np.all(np.abs(d1[differ] - d2[differ]) <= ulp)
    else:
        np.testing.assert_array_equal(d2, d1)
    # and against numpy: softmax over the rows of every column of the scaled, masked scores
    from gpu_util import TOL
    xs = np.where(np.tile(mask, (1, batch)) != 0, x.astype(np.float64) * scale, -np.inf)
    e = np.exp(xs - xs.max(axis=0, keepdims=True))
    want_y = e / e.sum(axis=0, keepdims=True)
    got_y = get(by2).reshape(x.shape, order="F")
    assert rel_fro(got_y, want_y) <= TOL[dt]
    g = dy.astype(np.float64)
    want_d = scale * np.where(np.tile(mask, (1, batch)) != 0, want_y * (g - (want_y * g).sum(axis=0, keepdims=True)), 0)
    assert rel_fro(get(bd2).reshape(x.shape, order="F"), want_d) <= TOL[dt] * 2


def test_scaled_masked_softmax_arguments(dev):
    t = dev.torch
    buf = t.zeros(256, device="cuda")
    p, q = c_void_p(buf.data_ptr()), c_void_p(buf.data_ptr() + 512)
    bad = [
        ("ginn_hip_scaled_masked_softmax_fwd", (dev.ctx, capi.F32, 8, 8, p, 1.0, q, 48, 0.0, q)),   # 48 does not divide 64
        ("ginn_hip_scaled_masked_softmax_fwd", (dev.ctx, capi.F32, 8, 8, p, 1.0, q, 64, 0.0, p)),   # y is x
        ("ginn_hip_scaled_masked_softmax_fwd", (dev.ctx, capi.F32, 8, 8, None, 1.0, q, 64, 0.0, q)),
        ("ginn_hip_scaled_masked_softmax_fwd", (dev.ctx, capi.F32, -8, 8, p, 1.0, q, 64, 0.0, q)),
        ("ginn_hip_scaled_masked_softmax_bwd", (dev.ctx, capi.F32, 8, 8, p, q, 1.0, q, 0, q)),      # empty mask
        ("ginn_hip_scaled_masked_softmax_bwd", (dev.ctx, capi.F32, 8, 8, p, q, 1.0, q, 64, p)),     # dx is dy
        ("ginn_hip_scaled_masked_softmax_bwd", (dev.ctx, 9, 8, 8, p, q, 1.0, q, 64, c_void_p(buf.data_ptr() + 768))),
    ]
    for name, args in bad:
        with pytest.raises(capi.GinnHipError):
            dev.lib.call(name, *args)
    dev.lib.call("ginn_hip_scaled_masked_softmax_fwd", dev.ctx, capi.F32, 0, 8, None, 1.0, None, 1, 0.0, None)
    dev.lib.call("ginn_hip_scaled_masked_softmax_bwd", dev.ctx, capi.F32, 8, 0, None, None, 1.0, None, 1, None)


# ---------------------------------------------------------------------------
# postponed folds of row sums
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("dt", DTYPES)
def test_postponed_folds_give_the_same_sums(dev, dt):
    """ginn_hip_defer_folds / ginn_hip_flush_folds: the second launch of every row
    reduction started meanwhile waits, the destinations keep their old values,
    one launch then folds all of them to the bits of the unpostponed calls; two
    folds into one destination are not put into one launch."""
    from gpu_util import round_to
    rng = np.random.default_rng(11)
    shapes = [(768, 520), (40, 33), (1024, 64)]
    xs = [round_to(rng.standard_normal(s), dt) for s in shapes]
    old = [round_to(rng.standard_normal(s[0]), dt) for s in shapes]

    def row_sums(postpone):
        outs = []
        for x, o in zip(xs, old):
            bx, px, _ = dev.put(x, dt)
            bo, po, _ = dev.put(o, dt)
            outs.append((bx, bo, px, po, x.shape))
        if postpone:
            dev.lib.call("ginn_hip_defer_folds", dev.ctx, 1)
        for bx, bo, px, po, (r, c) in outs:
            dev.lib.call("ginn_hip_row_sum", dev.ctx, dt, r, c, c_void_p(px), c_void_p(po), 1)
        if postpone:
            dev.lib.call("ginn_hip_defer_folds", dev.ctx, 0)
            n = ctypes.c_int(-1)
            dev.lib.call("ginn_hip_pending_folds", dev.ctx, ctypes.byref(n))
            assert n.value == len(shapes)
            for (bx, bo, px, po, (r, c)), o in zip(outs, old):   # nothing folded yet
                np.testing.assert_array_equal(dev.get(bo, (r,)), o)
            dev.lib.call("ginn_hip_flush_folds", dev.ctx)
            dev.lib.call("ginn_hip_pending_folds", dev.ctx, ctypes.byref(n))
            assert n.value == 0
        dev.sync()
        return [dev.get(bo, (r,)) for bx, bo, px, po, (r, c) in outs]

    plain, later = row_sums(False), row_sums(True)
    for a, b, x, o in zip(plain, later, xs, old):
        np.testing.assert_array_equal(b, a)
        from gpu_util import TOL
        assert rel_fro(a, x.astype(np.float64).sum(axis=1) + o) <= TOL[dt]

    # two sums into one destination: the second one folds the first before it queues itself
    bx, px, _ = dev.put(xs[0], dt)
    bo, po, _ = dev.put(np.zeros(shapes[0][0]), dt)
    dev.lib.call("ginn_hip_defer_folds", dev.ctx, 1)
    for _ in range(2):
        dev.lib.call("ginn_hip_row_sum", dev.ctx, dt, shapes[0][0], shapes[0][1], c_void_p(px), c_void_p(po), 1)
    n = ctypes.c_int(-1)
    dev.lib.call("ginn_hip_pending_folds", dev.ctx, ctypes.byref(n))
    assert n.value == 1
    dev.lib.call("ginn_hip_defer_folds", dev.ctx, 0)
    dev.sync()  # waits for the postponed fold as well
    once = round_to(xs[0].astype(np.float64).sum(axis=1), dt)
    assert rel_fro(dev.get(bo, (shapes[0][0],)), 2.0 * once) <= TOL[dt]
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_defer_folds", dev.ctx, 0)   # switched off more often than on


# ---------------------------------------------------------------------------
# GPT decoder layer through the host layer
# ---------------------------------------------------------------------------

def run_gpt(shim, dt, C, nh, B, T, V, seed, iters=1, wscale=0.02):
    from gpu_util import round_to
    rng = np.random.default_rng(seed)
    shapes = dict(ln1_g=(C,), ln1_b=(C,), Wk=(C, C), bk=(C,), Wq=(C, C), bq=(C,), Wv=(C, C), bv=(C,), Wp=(C, C),
                  bp=(C,), ln2_g=(C,), ln2_b=(C,), W1=(4 * C, C), b1=(4 * C,), W2=(C, 4 * C), b2=(C,), lnf_g=(C,),
                  lnf_b=(C,), Wh=(V, C), bh=(V,))
    params = {k: round_to(rng.standard_normal(s) * wscale, dt) for k, s in shapes.items()}
    x = round_to(rng.standard_normal((C, B, T)), dt)
    targets = rng.integers(0, V, B * T).astype(np.int32)
    f32 = lambda a: np.asfortranarray(a, dtype=np.float32)
    pin = [f32(params[k]) for k in N.GptBlockParams.NAMES]
    grads = [np.zeros(shapes[k], np.float32, order="F") for k in N.GptBlockParams.NAMES]
    dx = np.zeros((C, B, T), np.float32, order="F")
    loss = np.zeros(1, np.float32)
    ms, nodes = ctypes.c_float(0), ctypes.c_int(0)
    rc = shim.scenario_gpt_layer(
        dt, C, nh, B, T, V, f32(x).ctypes.data_as(FP), targets.ctypes.data_as(ctypes.POINTER(ctypes.c_int)),
        (FP * 20)(*[a.ctypes.data_as(FP) for a in pin]), iters, loss.ctypes.data_as(FP),
        (FP * 20)(*[a.ctypes.data_as(FP) for a in grads]), dx.ctypes.data_as(FP), ctypes.byref(ms),
        ctypes.byref(nodes))
    assert rc == 0, shim.scenario_last_error().decode()
    # no gradient that reset_grad() had only flagged was read or added to before its user overwrote it
    shim.scenario_timed_fills.restype = ctypes.c_long
    assert shim.scenario_timed_fills() == 0
    p64 = N.GptBlockParams(**{k: np.asfortranarray(v.astype(np.float64)) for k, v in params.items()})
    wloss, wgrads = N.gpt_layer_forward_backward(p64, np.asfortranarray(x.astype(np.float64)), targets, nh)
    got = dict(zip(N.GptBlockParams.NAMES, grads))
    got["x"] = dx
    return float(loss[0]), got, wloss, wgrads, ms.value


def grad_errors(got, want):
    """Relative Frobenius error per gradient.  The key bias has an identically
    zero gradient (a constant added to every key's score cancels in the
    softmax), so it is measured against the query bias gradient's size."""
    errs = {}
    for name, w in want.items():
        w = np.asarray(w).reshape(got[name].shape, order="F")
        if name == "bk":
            errs[name] = float(np.linalg.norm(got[name] - w) / np.linalg.norm(want["bq"]))
        else:
            errs[name] = rel_fro(got[name], w)
    return errs


@pytest.mark.parametrize("C,nh,B,T,V", [(12, 3, 2, 5, 11), (64, 4, 3, 33, 50), (128, 2, 2, 64, 97)])
def test_gpt_layer_fp32(shim, C, nh, B, T, V):
    loss, got, wloss, want, _ = run_gpt(shim, capi.F32, C, nh, B, T, V, seed=C, wscale=0.2)
    assert abs(loss - wloss) <= 1e-4 * abs(wloss)
    errs = grad_errors(got, want)
    assert max(errs.values()) <= 1e-4, errs


@pytest.mark.parametrize("rule", ["sgd", "adam"])
def test_gpt_layer_training_steps(shim, rule):
    """Whole training steps: every pass ends with Updater::update over all 20
    weights (ginn/update/update.h:34-46; one launch here).  The loss and the
    gradients of the fourth pass -- after three updates -- against the oracle's
    own three steps, and the loss has to fall."""
    from oracle import update as U
    from gpu_util import round_to
    C, nh, B, T, V, lr, clip = 64, 4, 3, 33, 50, (0.05 if rule == "sgd" else 5e-3), 1.0
    shim.scenario_set_training(0 if rule == "sgd" else 1, ctypes.c_float(lr), ctypes.c_float(clip))
    try:
        loss, got, first_loss, _, _ = run_gpt(shim, capi.F32, C, nh, B, T, V, seed=C, iters=3, wscale=0.2)
    finally:
        shim.scenario_set_training(-1, ctypes.c_float(0), ctypes.c_float(0))
    # the oracle's trajectory from the same start (run_gpt's generator, same seed)
    rng = np.random.default_rng(C)
    shapes = dict(ln1_g=(C,), ln1_b=(C,), Wk=(C, C), bk=(C,), Wq=(C, C), bq=(C,), Wv=(C, C), bv=(C,), Wp=(C, C),
                  bp=(C,), ln2_g=(C,), ln2_b=(C,), W1=(4 * C, C), b1=(4 * C,), W2=(C, 4 * C), b2=(C,), lnf_g=(C,),
                  lnf_b=(C,), Wh=(V, C), bh=(V,))
    params = {k: round_to(rng.standard_normal(sh) * 0.2, capi.F32) for k, sh in shapes.items()}
    x = round_to(rng.standard_normal((C, B, T)), capi.F32)
    targets = rng.integers(0, V, B * T).astype(np.int32)
    adam = U.Adam(lr=lr, clip=clip)
    for step in range(4):
        p64 = N.GptBlockParams(**{k: np.asfortranarray(v.astype(np.float64)) for k, v in params.items()})
        wloss, wgrads = N.gpt_layer_forward_backward(p64, np.asfortranarray(x.astype(np.float64)), targets, nh)
        if step == 3:
            break
        for i, k in enumerate(N.GptBlockParams.NAMES):
            g = np.asarray(wgrads[k], np.float32).reshape(params[k].shape, order="F")
            if rule == "sgd":
                params[k], _ = U.sgd_update(params[k], g, lr, clip)
            else:
                params[k], _ = adam.update(params[k], g, i)
    assert abs(loss - wloss) <= 2e-4 * abs(wloss)
    assert wloss < first_loss and loss < first_loss
    errs = grad_errors(got, wgrads)
    assert max(errs.values()) <= 1e-3, errs


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
def test_gpt_layer_16bit_small(shim, dt):
    loss, got, wloss, want, _ = run_gpt(shim, dt, 128, 4, 2, 64, 301, seed=3, wscale=0.1)
    assert abs(loss - wloss) <= 2e-2 * abs(wloss)
    errs = grad_errors(got, want)
    print({k: round(v, 4) for k, v in errs.items()})
    # every gradient of the chain (a dozen 16-bit roundings deep) stays inside the single-product bound
    assert max(errs.values()) <= 2e-2, errs


def test_gpt_layer_bf16_full_config(shim):
    """d_model 768, 12 heads, sequence 512, batch 8, MLP 3072, vocabulary 8192; weights N(0, 0.02)."""
    loss, got, wloss, want, ms = run_gpt(shim, capi.BF16, 768, 12, 8, 512, 8192, seed=5, iters=2)
    print(f"gpt layer fwd+bwd {ms:.2f} ms, loss {loss:.4f} vs {wloss:.4f}")
    assert abs(loss - wloss) <= 2e-2 * abs(wloss)
    errs = grad_errors(got, want)
    print({k: round(v, 4) for k, v in errs.items()})
    assert max(errs.values()) <= 2e-2, errs


@pytest.mark.parametrize("mode", [2, 6, 14])
@pytest.mark.parametrize("dt,tol", [(capi.F32, 1e-4), (capi.BF16, 2e-2)])
def test_gpt_layer_level_executor(shim, dt, tol, mode):
    """The same layer through the level executor (2) and with the executor
    frozen after its first pass (6): the gradients are reset by one zero-fill
    launch, equal-shaped element-wise nodes of one height share launches; same
    oracle, same tolerance.  Against node-by-node execution only the order in
    which the users of a node add into its gradient differs (rounding level)."""
    args = (dt, 128, 4, 2, 64, 301)
    shim.scenario_set_executor(mode)
    try:
        loss, got, wloss, want, _ = run_gpt(shim, *args, seed=3, iters=2, wscale=0.1)
    finally:
        shim.scenario_set_executor(0)
    assert abs(loss - wloss) <= tol * abs(wloss)
    errs = grad_errors(got, want)
    assert max(errs.values()) <= tol, errs
    ploss, plain, _, _, _ = run_gpt(shim, *args, seed=3, iters=2, wscale=0.1)
    assert loss == ploss  # forward: the same arithmetic per element
    for name in plain:
        scale = np.linalg.norm(plain["bq" if name == "bk" else name])
        assert np.linalg.norm(got[name] - plain[name]) <= (1e-5 if dt == capi.F32 else 5e-3) * scale, name


def test_multi_zero(dev):
    """Regions of every size and alignment, one launch; bytes around them stay."""
    t = dev.torch
    rng = np.random.default_rng(11)
    sizes = [0, 1, 3, 15, 16, 17, 64, 1000, 4096, 65537, 1 << 20]
    offs = [0, 1, 2, 4, 8, 16, 3, 0, 5, 0, 16]
    pad = 32
    bufs, ptrs = [], []
    for n, o in zip(sizes, offs):
        b = t.from_numpy(rng.integers(1, 255, n + o + pad, dtype=np.uint8)).to("cuda")
        bufs.append(b)
        ptrs.append(b.data_ptr() + o)
    before = [b.cpu().numpy().copy() for b in bufs]
    tp = t.tensor(ptrs, dtype=t.int64, device="cuda")
    tb = t.tensor(sizes, dtype=t.int64, device="cuda")
    dev.lib.call("ginn_hip_multi_zero", dev.ctx, len(sizes), c_void_p(tp.data_ptr()), c_void_p(tb.data_ptr()),
                 max(sizes))
    dev.sync()
    for b, ref, n, o in zip(bufs, before, sizes, offs):
        got = b.cpu().numpy()
        assert not got[o:o + n].any()
        np.testing.assert_array_equal(got[:o], ref[:o])
        np.testing.assert_array_equal(got[o + n:], ref[o + n:])
    dev.lib.call("ginn_hip_multi_zero", dev.ctx, 0, None, None, 0)  # nothing to do
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_multi_zero", dev.ctx, 2, None, c_void_p(tb.data_ptr()), 16)


def test_argument_validation(dev):
    """Bad shapes, dtypes and pointers are refused before any launch."""
    t = dev.torch
    buf = t.zeros(64, device="cuda")
    p = c_void_p(buf.data_ptr())
    bad = [
        ("ginn_hip_layernorm_fwd", (dev.ctx, capi.F32, -1, 4, p, 1e-8, p, p)),
        ("ginn_hip_layernorm_fwd", (dev.ctx, capi.F32, 4, 4, None, 1e-8, p, p)),
        ("ginn_hip_layernorm_fwd", (dev.ctx, 7, 4, 4, p, 1e-8, p, p)),
        ("ginn_hip_layernorm_bwd", (dev.ctx, capi.F32, 4, 4, p, p, None, p)),
        ("ginn_hip_cwise_prod_add_fwd", (dev.ctx, capi.F32, 4, -4, p, p, p, 0.0, 1, p)),
        ("ginn_hip_cwise_prod_add_bwd", (dev.ctx, capi.F32, 4, 4, None, p, p, 0.0, 1, p, p, p)),
        ("ginn_hip_mask_fill", (dev.ctx, capi.F32, 4, 4, None, 0.0, p)),
        ("ginn_hip_upper_tri", (dev.ctx, capi.F32, -3, p)),
        ("ginn_hip_upper_tri", (dev.ctx, 9, 3, p)),
    ]
    for name, args in bad:
        with pytest.raises(capi.GinnHipError):
            dev.lib.call(name, *args)
    # empty extents are valid no-ops
    dev.lib.call("ginn_hip_layernorm_fwd", dev.ctx, capi.F32, 0, 4, None, 1e-8, None, None)
    dev.lib.call("ginn_hip_upper_tri", dev.ctx, capi.F32, 0, None)
    dev.lib.call("ginn_hip_mask_fill", dev.ctx, capi.F32, 0, 4, None, 0.0, None)
    dims = (ctypes.c_longlong * 2)(0, 4)
    dev.lib.call("ginn_hip_permute", dev.ctx, capi.F32, 2, dims, (ctypes.c_int * 2)(1, 0), None, None, 0)


@pytest.mark.parametrize("dt", DTYPES)
def test_multi_apply(dev, dt):
    """Many equal-sized elementwise operations in one launch: every kind,
    assigning and accumulating, against numpy on each operation."""
    from gpu_util import TOL, round_to, torch_dtype
    t = dev.torch
    rng = np.random.default_rng(dt)
    count, n = 37, 300
    a = round_to(rng.standard_normal((count, n)), dt)
    b = round_to(rng.standard_normal((count, n)), dt)
    c = round_to(rng.standard_normal((count, n)), dt)
    base = round_to(rng.standard_normal((count, n)), dt)
    tdt = torch_dtype(dt)
    A, B, C = (t.from_numpy(x).to("cuda").to(tdt) for x in (a, b, c))
    es = A.element_size()

    def table(x):
        # operations live at arbitrary places: every second row of a wider buffer
        return t.tensor([x.data_ptr() + i * n * es for i in range(count)], dtype=t.int64, device="cuda")

    ta, tb, tc = table(A), table(B), table(C)
    cases = [
        (0, 0, 0, 1.5, (), lambda: np.full((count, n), 1.5)),
        (1, 0, 0, 0.0, (ta,), lambda: a), (1, 0, 1, 0.0, (ta, tb), lambda: base + a + b),
        (1, 0, 0, 0.0, (ta, tb, tc), lambda: a + b + c), (2, 0, 1, 0.0, (ta, tb), lambda: base + a * b),
        (3, N.TANH, 0, 0.0, (ta,), lambda: np.tanh(a)), (3, N.SIGMOID, 0, 0.0, (ta,), lambda: 1 / (1 + np.exp(-a))),
        (4, N.TANH, 1, 0.0, (ta, tb, tc), lambda: base + (1 - c * c) * a),
        (4, N.RELU, 0, 0.0, (ta, tb, tc), lambda: a * (c > 0)),
    ]
    for kind, act, acc, value, srcs, want in cases:
        D = t.from_numpy(base).to("cuda").to(tdt)
        td = table(D)
        ptrs = [c_void_p(s.data_ptr()) for s in srcs] + [None] * (3 - len(srcs))
        dev.lib.call("ginn_hip_multi_apply", dev.ctx, dt, kind, act, acc, value, n, count, c_void_p(td.data_ptr()),
                     *ptrs)
        dev.sync()
        got = D.float().cpu().numpy()
        assert rel_fro(got, round_to(want(), dt) if kind in (0,) else want()) <= TOL[dt], (kind, act, acc)
    with pytest.raises(capi.GinnHipError):  # softmax is not elementwise
        dev.lib.call("ginn_hip_multi_apply", dev.ctx, dt, 3, N.SOFTMAX, 0, 0.0, n, count, c_void_p(ta.data_ptr()),
                     c_void_p(ta.data_ptr()), None, None)
    with pytest.raises(capi.GinnHipError):  # a product needs two sources
        dev.lib.call("ginn_hip_multi_apply", dev.ctx, dt, 2, 0, 0, 0.0, n, count, c_void_p(ta.data_ptr()),
                     c_void_p(ta.data_ptr()), None, None)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [1, 64, 1000, 16384, 16385, 100000, 3000001])
def test_sum_all(dev, dt, n):
    """SumNode / MeanNode forward (ginn/node/reduce.h): one block for a short
    vector, per-block partials and a fold for a long one."""
    from gpu_util import round_to, torch_dtype
    t = dev.torch
    rng = np.random.default_rng(n)
    x = round_to(rng.standard_normal(n) + 0.25, dt)
    X = t.from_numpy(x).to("cuda").to(torch_dtype(dt))
    D = t.full((1,), float("nan"), device="cuda", dtype=torch_dtype(dt))
    scale = 1.0 / n
    dev.lib.call("ginn_hip_sum_all", dev.ctx, dt, n, c_void_p(X.data_ptr()), scale, c_void_p(D.data_ptr()))
    dev.sync()
    want = float(x.astype(np.float64).sum() * scale)
    got = float(D.float().cpu().numpy()[0])
    # fp32 accumulation of n values, then one rounding to the storage type
    tol = {capi.F32: 2e-5, capi.F16: 2e-3, capi.BF16: 1e-2}[dt]
    assert abs(got - want) <= tol * max(1.0, abs(want)), (got, want)


def test_multi_mixed(dev):
    """Operations of different kinds, lengths and scalar types in ONE launch:
    each record of the table against numpy.  Lengths cover the 16-byte path
    (multiples of 8, aligned), the element-wise path (odd lengths, operands
    shifted off 16 bytes) and an operation far longer than the others (the
    launch is sized for it; the others' extra blocks find nothing to do)."""
    import struct
    from gpu_util import TOL, round_to, torch_dtype
    t = dev.torch
    rng = np.random.default_rng(11)
    keep, records, checks = [], [], []

    def operand(x, dt, shift=0):
        buf = t.zeros(x.size + 8 + shift, dtype=torch_dtype(dt), device="cuda")
        buf[shift:shift + x.size] = t.from_numpy(x).to("cuda").to(torch_dtype(dt))
        keep.append(buf)
        return buf, buf.data_ptr() + shift * buf.element_size()

    def add(dt, kind, act, acc, value, n, nsrc, want, shift=0):
        srcs = [round_to(rng.standard_normal(n), dt) for _ in range(nsrc)]
        if kind == 4:
            srcs[2] = round_to(np.tanh(srcs[1]), dt) if act == N.TANH else srcs[2]
        base = round_to(rng.standard_normal(n), dt)
        ptrs = [operand(x, dt, shift)[1] for x in srcs] + [0] * (3 - nsrc)
        dbuf, dptr = operand(base, dt, shift)
        records.append(struct.pack("<iiiifiQQQQQ", dt, kind, act, acc, value, 0, n, dptr, *ptrs))
        expect = want(*srcs) + (base if acc else 0)
        checks.append((dbuf, shift, n, expect, dt, (dt, kind, act, acc, n)))

    for dt in DTYPES:
        add(dt, 0, 0, 0, 2.5, 64, 0, lambda: np.full(64, 2.5))
        add(dt, 0, 0, 1, -1.0, 33, 0, lambda: np.full(33, -1.0), shift=1)
        add(dt, 1, 0, 0, 0.0, 256, 1, lambda a: a)
        add(dt, 1, 0, 1, 0.0, 1024, 2, lambda a, b: a + b)
        add(dt, 1, 0, 0, 0.0, 7, 3, lambda a, b, c: a + b + c, shift=3)
        add(dt, 2, 0, 1, 0.0, 256, 2, lambda a, b: a * b)
        add(dt, 3, N.TANH, 0, 0.0, 1000, 1, np.tanh)
        add(dt, 3, N.SIGMOID, 0, 0.0, 255, 1, lambda a: 1 / (1 + np.exp(-a)))
        add(dt, 4, N.TANH, 1, 0.0, 512, 3, lambda dy, x, y: (1 - y * y) * dy)
        add(dt, 4, N.RELU, 0, 0.0, 100, 3, lambda dy, x, y: dy * (y > 0), shift=2)
    add(capi.BF16, 3, N.GELU, 0, 0.0, 3 * 1024 * 1024, 1,
        lambda a: N.nonlin_forward(N.GELU, a.astype(np.float64)))  # the longest by far
    blob = b"".join(records)
    assert len(blob) == 64 * len(records)
    table = t.frombuffer(bytearray(blob), dtype=t.uint8).to("cuda")
    max_n = 3 * 1024 * 1024
    dev.lib.call("ginn_hip_multi_mixed", dev.ctx, len(records), c_void_p(table.data_ptr()), max_n)
    dev.sync()
    for dbuf, shift, n, expect, dt, what in checks:
        got = dbuf[shift:shift + n].float().cpu().numpy()
        assert rel_fro(got, expect) <= TOL[dt], what
        # nothing written around the operation
        assert float(dbuf[shift + n:].float().abs().sum()) == 0.0 and float(dbuf[:shift].float().abs().sum()) == 0.0, what
    # nothing to do
    dev.lib.call("ginn_hip_multi_mixed", dev.ctx, 0, None, 0)
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_multi_mixed", dev.ctx, 3, None, 8)
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_multi_mixed", dev.ctx, 70000, c_void_p(table.data_ptr()), 8)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n,count", [(1024, 256), (7, 3), (300, 1), (64, 1000), (5, 0)])
def test_multi_reduce(dev, dt, n, count):
    from gpu_util import TOL, round_to, torch_dtype
    t = dev.torch
    rng = np.random.default_rng(n + count)
    srcs = np.ascontiguousarray(round_to(rng.standard_normal((max(count, 1), n)), dt))  # one source per row
    base = round_to(rng.standard_normal(n), dt)
    S = t.from_numpy(srcs).to("cuda").to(torch_dtype(dt))
    table = t.tensor([S.data_ptr() + i * n * S.element_size() for i in range(count)] or [0], dtype=t.int64,
                     device="cuda")
    for acc in (0, 1):
        D = t.from_numpy(base).to("cuda").to(torch_dtype(dt))
        dev.lib.call("ginn_hip_multi_reduce", dev.ctx, dt, n, count, c_void_p(table.data_ptr()),
                     c_void_p(D.data_ptr()), acc)
        dev.sync()
        want = srcs[:count].astype(np.float64).sum(axis=0) + (base if acc else 0)
        got = D.float().cpu().numpy()
        if count == 0 and not acc:
            assert not got.any()
        else:
            assert np.linalg.norm(got - want) <= TOL[dt] * max(np.linalg.norm(want), 1e-3) * 2


def test_multi_chain(dev):
    """Chains of dependent operations in one launch: per chain a = tanh(x) and
    b = sigmoid(x) (one stage), p = a * b (next stage), acc += p, acc += p
    (two more stages on one destination); lengths on both sides of the limit up
    to which a wave takes an operation alone, odd lengths and shifted operands
    for the element-wise path, and one chain of more records than fit the
    kernel's record buffer (150 fills in one stage, then sums of them)."""
    import struct
    from gpu_util import round_to, torch_dtype
    t = dev.torch
    rng = np.random.default_rng(5)
    keep, records, ranges, checks = [], [], [], []

    def operand(x, dt, shift=0):
        buf = t.zeros(x.size + 8 + shift, dtype=torch_dtype(dt), device="cuda")
        buf[shift:shift + x.size] = t.from_numpy(np.asarray(x, np.float32)).to("cuda").to(torch_dtype(dt))
        keep.append(buf)
        return buf, buf.data_ptr() + shift * buf.element_size()

    def rec(dt, kind, act, acc, value, stage, n, dst, *srcs):
        srcs = list(srcs) + [0] * (3 - len(srcs))
        records.append(struct.pack("<iiiifiQQQQQ", dt, kind, act, acc, value, stage, n, dst, *srcs))

    for dt, n, shift in [(capi.F32, 8, 0), (capi.F32, 255, 1), (capi.F16, 1000, 0), (capi.BF16, 256, 0),
                         (capi.F32, 5000, 0), (capi.F32, 4096, 0), (capi.F16, 33, 3)] * 6:
        x = round_to(rng.standard_normal(n), dt)
        base = round_to(rng.standard_normal(n), dt)
        _, px = operand(x, dt, shift)
        _, pa = operand(np.zeros(n), dt, shift)
        _, pb = operand(np.zeros(n), dt, shift)
        _, pp = operand(np.zeros(n), dt, shift)
        bacc, pacc = operand(base, dt, shift)
        first = len(records)
        rec(dt, 3, N.TANH, 0, 0.0, 0, n, pa, px)
        rec(dt, 3, N.SIGMOID, 0, 0.0, 0, n, pb, px)
        rec(dt, 2, 0, 0, 0.0, 1, n, pp, pa, pb)
        rec(dt, 1, 0, 1, 0.0, 2, n, pacc, pp)
        rec(dt, 1, 0, 1, 0.0, 3, n, pacc, pp)
        ranges.append((first, len(records) - first))
        a = round_to(np.tanh(x.astype(np.float64)), dt).astype(np.float64)
        b = round_to(1 / (1 + np.exp(-x.astype(np.float64))), dt).astype(np.float64)
        prod = round_to(a * b, dt).astype(np.float64)
        checks.append((bacc, shift, n, base + 2 * prod, dt))
    # a chain longer than the record buffer: 150 fills, then pairwise sums of them into one vector
    n = 64
    fills = [operand(np.zeros(n), capi.F32)[1] for _ in range(150)]
    btot, ptot = operand(np.zeros(n), capi.F32)
    first = len(records)
    for i, pf in enumerate(fills):
        rec(capi.F32, 0, 0, 0, float(i), 0, n, pf)
    for i in range(0, 150, 2):
        rec(capi.F32, 1, 0, 1, 0.0, 1 + i // 2, n, ptot, fills[i], fills[i + 1])
    ranges.append((first, len(records) - first))
    checks.append((btot, 0, n, np.full(n, float(sum(range(150)))), capi.F32))

    blob = b"".join(records)
    table = t.frombuffer(bytearray(blob), dtype=t.uint8).to("cuda")
    rblob = b"".join(struct.pack("<II", f, c) for f, c in ranges)
    rtable = t.frombuffer(bytearray(rblob), dtype=t.uint8).to("cuda")
    dev.lib.call("ginn_hip_multi_chain", dev.ctx, len(ranges), c_void_p(rtable.data_ptr()), c_void_p(table.data_ptr()))
    dev.sync()
    tol = {capi.F32: 1e-5, capi.F16: 4e-3, capi.BF16: 3e-2}
    for dbuf, shift, n, expect, dt in checks:
        got = dbuf[shift:shift + n].float().cpu().numpy()
        assert rel_fro(got, expect) <= tol[dt], (dt, n, shift)
    dev.lib.call("ginn_hip_multi_chain", dev.ctx, 0, None, None)
    with pytest.raises(capi.GinnHipError):
        dev.lib.call("ginn_hip_multi_chain", dev.ctx, 3, None, None)


def test_multi_chain_overlapping_operands(dev):
    """Chains whose records read and write overlapping memory in every way a graph can ask for, each checked
    against the records applied one after the other on the host: the element-wise part of a recurrent cell (a
    1024-element sum, four slices of it copied, nonlinearities, products, a sum, a result written into a column
    of a table), lengths that are no multiples of the workgroup, in-place and accumulating records, a record that
    writes over an earlier record's source, operands that are shifted against each other (a source that overlaps
    an earlier destination at another offset, or reaches beyond it into what memory held before)."""
    import struct
    t = dev.torch
    rng = np.random.default_rng(17)
    SUM, PROD, FWD, BWD, FILL = 1, 2, 3, 4, 0
    arena = t.zeros(1 << 20, dtype=t.float32, device="cuda")  # one allocation: every offset below is in floats
    base_ptr = arena.data_ptr()
    assert base_ptr % 1024 == 0
    initial = np.zeros(1 << 20, np.float32)
    cursor = [0]
    records, ranges = [], []

    def alloc(n, shift=0, init=None):
        off = (cursor[0] + 255) // 256 * 256 + shift  # on the grid of 256 floats, plus `shift` floats
        cursor[0] = off + n + 256
        if init is not None:
            initial[off:off + n] = init
        return off

    def rec(kind, act, acc, value, stage, n, dst, *srcs):
        srcs = list(srcs) + [None] * (3 - len(srcs))
        ptrs = [0 if o is None else base_ptr + 4 * o for o in srcs]
        records.append((struct.pack("<iiiifiQQQQQ", capi.F32, kind, act, acc, value, stage, n, base_ptr + 4 * dst, *ptrs),
                        (kind, act, acc, value, n, dst, srcs)))

    def begin():
        return len(records)

    def end(first):
        ranges.append((first, len(records) - first))

    def rnd(n):
        return rng.standard_normal(n).astype(np.float32)

    # 1. the element-wise part of an LSTM step, several chains of it
    for _ in range(6):
        H = 256
        prod, bias, c_prev = alloc(4 * H, init=rnd(4 * H)), alloc(4 * H, init=rnd(4 * H)), alloc(H, init=rnd(H))
        z = alloc(4 * H)
        gates = [alloc(H) for _ in range(4)]
        acts = [alloc(H) for _ in range(4)]
        fc, ig, c, tc, h = (alloc(H) for _ in range(5))
        out = alloc(H, shift=128)  # a column of a table: 512 bytes off the grid
        f0 = begin()
        rec(SUM, 0, 0, 0.0, 0, 4 * H, z, prod, bias)
        for q in range(4):
            rec(SUM, 0, 0, 0.0, 1, H, gates[q], z + H * [3, 1, 0, 2][q])
        for q in range(4):
            rec(FWD, N.TANH if q == 3 else N.SIGMOID, 0, 0.0, 2, H, acts[q], gates[q])
        rec(PROD, 0, 0, 0.0, 3, H, fc, acts[1], c_prev)
        rec(PROD, 0, 0, 0.0, 3, H, ig, acts[2], acts[3])
        rec(SUM, 0, 0, 0.0, 4, H, c, fc, ig)
        rec(FWD, N.TANH, 0, 0.0, 5, H, tc, c)
        rec(PROD, 0, 0, 0.0, 6, H, h, acts[0], tc)
        rec(SUM, 0, 0, 0.0, 7, H, out, h)
        end(f0)
    # 2. lengths that fill no block, in-place and accumulating records, the gradient of a nonlinearity
    for n in (4, 200, 255, 257, 1000, 1024):
        x, y, g = alloc(n, init=rnd(n)), alloc(n), alloc(n, init=rnd(n))
        acc = alloc(n, init=rnd(n))
        f0 = begin()
        rec(FWD, N.TANH, 0, 0.0, 0, n, y, x)
        rec(BWD, N.TANH, 0, 0.0, 1, n, g, g, x, y)      # in place: g = g * (1 - y^2)
        rec(SUM, 0, 1, 0.0, 2, n, acc, g)                # acc += g
        rec(PROD, 0, 1, 0.0, 3, n, acc, acc, y)          # acc += acc * y (reads what it adds to)
        rec(FILL, 0, 0, 2.5, 4, n, x)                    # writes over a source of stage 0
        rec(SUM, 0, 0, 0.0, 5, n, y, x, acc)             # y = 2.5 + acc, over an earlier destination
        end(f0)
    # 3. all operands at the same offset from the grid
    for shift in (1, 77):
        n = 300
        x, y, w = alloc(n, shift, rnd(n)), alloc(n, shift), alloc(n, shift)
        f0 = begin()
        rec(FWD, N.SIGMOID, 0, 0.0, 0, n, y, x)
        rec(PROD, 0, 0, 0.0, 1, n, w, y, x)
        rec(SUM, 0, 0, 0.0, 2, n, y, w, y)
        end(f0)
    # 4. a source overlapping an earlier destination at another offset: values pass between threads
    n = 256
    x, y = alloc(n + 8, init=rnd(n + 8)), alloc(n + 8, init=rnd(n + 8))
    w = alloc(n)
    f0 = begin()
    rec(FWD, N.TANH, 0, 0.0, 0, n, y, x)
    rec(SUM, 0, 0, 0.0, 1, n, w, y + 4, x + 4)  # reads y shifted by four elements
    end(f0)
    # 5. a source that reaches beyond the destination it overlaps
    x, y, w = alloc(256, init=rnd(256)), alloc(256, init=rnd(256)), alloc(256)
    f0 = begin()
    rec(FWD, N.RELU, 0, 0.0, 0, 200, y, x)
    rec(SUM, 0, 0, 0.0, 1, 256, w, y, x)  # elements 200 .. 255 of y are what memory held
    end(f0)
    # 6. a record that writes over the source of an earlier one at another offset
    x, y = alloc(512, init=rnd(512)), alloc(256)
    f0 = begin()
    rec(FWD, N.TANH, 0, 0.0, 0, 256, y, x)
    rec(FILL, 0, 0, -1.0, 1, 256, x + 128)
    rec(SUM, 0, 0, 0.0, 2, 256, y, y, x)
    end(f0)
    # the records applied one after the other on the host, in double precision with fp32 results
    def act(code, v):
        return {N.TANH: np.tanh, N.SIGMOID: lambda u: 1 / (1 + np.exp(-u)), N.RELU: lambda u: np.maximum(u, 0)}[code](v)

    assert cursor[0] < initial.size
    host = initial.copy()
    for _, (kind, a, acc, value, n, dst, srcs) in records:
        ins = [None if o is None else host[o:o + n].astype(np.float64) for o in srcs]
        if kind == FILL:
            v = np.full(n, value)
        elif kind == SUM:
            v = sum(i for i in ins if i is not None)
        elif kind == PROD:
            v = ins[0] * ins[1]
        elif kind == FWD:
            v = act(a, ins[0])
        else:
            assert a == N.TANH
            v = ins[0] * (1 - ins[2] ** 2)
        if acc:
            v = v + host[dst:dst + n]
        host[dst:dst + n] = v.astype(np.float32)

    table = t.frombuffer(bytearray(b"".join(r for r, _ in records)), dtype=t.uint8).to("cuda")
    rtable = t.frombuffer(bytearray(b"".join(struct.pack("<II", f, c) for f, c in ranges)), dtype=t.uint8).to("cuda")
    touched = np.zeros(initial.size, bool)
    for _, (_, _, _, _, n, dst, _) in records:
        touched[dst:dst + n] = True
    for _ in range(2):  # twice from the same start
        arena.copy_(t.from_numpy(initial))
        dev.lib.call("ginn_hip_multi_chain", dev.ctx, len(ranges), c_void_p(rtable.data_ptr()), c_void_p(table.data_ptr()))
        dev.sync()
        got = arena.cpu().numpy()
        for first, count in ranges:
            for _, (kind, a, acc, value, n, dst, srcs) in records[first:first + count]:
                np.testing.assert_allclose(got[dst:dst + n], host[dst:dst + n], rtol=3e-5, atol=3e-6,
                                           err_msg=f"chain at record {first}, destination {dst}, n {n}")
        np.testing.assert_array_equal(got[~touched], initial[~touched])  # nothing else was written
