"""GPU parity of ginn_hip_gemm / ginn_hip_gemm_strided_batched against the CPU
oracle on the same seeded inputs (protocol of the reference's CPU-vs-GPU
check, test/check_node.h:27-121).  Tolerances: fp32 <= 1e-4, fp16 / bf16
<= 2e-2 relative Frobenius error against the fp64-accumulating oracle."""
import ctypes

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi
from oracle import cgemm

pytestmark = pytest.mark.gpu

DTYPES = [capi.F32, capi.F16, capi.BF16]
LAYOUTS = [(0, 0), (0, 1), (1, 0), (1, 1)]


@pytest.fixture(scope="module")
def dev():
    from gpu_util import Dev
    d = Dev()
    yield d
    d.close()


def run_case(dev, dt, op_a, op_b, m, n, k, beta, pad=0, offset=0, seed=0):
    from gpu_util import TOL, TIGHT, round_to, stored
    rng = np.random.default_rng(seed)
    scale = 1.0 / np.sqrt(max(k, 1))
    A = round_to(rng.standard_normal((m, k)) * scale, dt)
    B = round_to(rng.standard_normal((k, n)), dt)
    C0 = round_to(rng.standard_normal((m, n)), dt)
    As, Bs = stored(A, op_a), stored(B, op_b)
    ba, pa, lda = dev.put(As, dt, pad, offset)
    bb, pb, ldb = dev.put(Bs, dt, pad, offset)
    bc, pc, ldc = dev.put(C0, dt, pad, offset)
    dev.gemm(dt, op_a, op_b, m, n, k, pa, lda, pb, ldb, beta, pc, ldc)
    dev.sync()
    got = dev.get(bc, (m, n), ldc, offset)
    want = cgemm.gemm(As, Bs, op_a, op_b, beta=beta, C=C0 if beta else None, kind="f64acc")
    err = rel_fro(got, want)
    assert np.isfinite(got).all()
    assert err <= TOL[dt], f"official tolerance: {err}"
    assert err <= TIGHT[dt], f"regression bound: {err}"
    if pad:
        # The padding rows of C (NaN on upload) must be untouched.
        raw = bc[offset:offset + n * ldc].float().cpu().numpy().reshape(n, ldc)
        assert np.isnan(raw[:, m:]).all()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", LAYOUTS)
def test_reference_prod_golden(dev, golden, dt, op_a, op_b):
    # test/nodes.cu.cpp:1023-1041 with its Real / Half tolerances.
    from conftest import farr
    from gpu_util import stored
    g = golden["prod"]
    W, V, WV = farr(g["W"], np.float32), farr(g["V"], np.float32), farr(g["WV"], np.float32)
    ba, pa, lda = dev.put(stored(W, op_a), dt)
    bb, pb, ldb = dev.put(stored(V, op_b), dt)
    bc, pc, ldc = dev.put(np.zeros((2, 2), np.float32), dt)
    dev.gemm(dt, op_a, op_b, 2, 2, 3, pa, lda, pb, ldb, 0.0, pc, ldc)
    dev.sync()
    # Real 1e-6 and Half 1e-2 are the reference's; bf16 (not in the reference)
    # carries 8 mantissa bits, hence 3e-2.
    eps = {capi.F32: 1e-6, capi.F16: 1e-2, capi.BF16: 3e-2}[dt]
    np.testing.assert_allclose(dev.get(bc, (2, 2)), WV, rtol=eps)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", LAYOUTS)
@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (3, 5, 7), (64, 64, 64), (65, 63, 33), (128, 128, 128),
                                   (200, 136, 72), (129, 257, 100), (10, 64, 512), (512, 64, 784),
                                   # fp32: one launch with K split inside the workgroup, up to its limits
                                   # (256 tiles of 32 x 32, K = 2048) and just beyond
                                   (33, 31, 36), (1024, 256, 384), (384, 250, 1024), (500, 500, 1000),
                                   (96, 40, 1028), (256, 64, 2048), (130, 100, 1900), (128, 64, 2052),
                                   # ... on 16 x 16 tiles (few large tiles, a long sum), ragged edges
                                   (384, 120, 1024), (50, 19, 520), (17, 250, 1000)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_small_shapes(dev, dt, op_a, op_b, m, n, k, beta):
    run_case(dev, dt, op_a, op_b, m, n, k, beta, seed=m * 7 + n * 3 + k)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", LAYOUTS)
@pytest.mark.parametrize("pad,offset", [(3, 0), (0, 1), (8, 8), (5, 3)])
def test_leading_dimension_and_alignment(dev, dt, op_a, op_b, pad, offset):
    run_case(dev, dt, op_a, op_b, 96, 72, 40, 1.0, pad=pad, offset=offset, seed=pad * 10 + offset)


@pytest.mark.parametrize("dt", DTYPES)
def test_beta_zero_ignores_c(dev, dt):
    from gpu_util import round_to
    rng = np.random.default_rng(1)
    A = round_to(rng.standard_normal((40, 24)), dt)
    B = round_to(rng.standard_normal((24, 56)), dt)
    ba, pa, lda = dev.put(A, dt)
    bb, pb, ldb = dev.put(B, dt)
    bc, pc, ldc = dev.put(np.full((40, 56), np.nan, np.float32), dt)
    dev.gemm(dt, 0, 0, 40, 56, 24, pa, lda, pb, ldb, 0.0, pc, ldc)
    dev.sync()
    assert np.isfinite(dev.get(bc, (40, 56))).all()


@pytest.mark.parametrize("dt", DTYPES)
def test_general_beta(dev, dt):
    from gpu_util import TIGHT, round_to
    rng = np.random.default_rng(2)
    A = round_to(rng.standard_normal((70, 30)), dt)
    B = round_to(rng.standard_normal((30, 50)), dt)
    C0 = round_to(rng.standard_normal((70, 50)), dt)
    ba, pa, lda = dev.put(A, dt)
    bb, pb, ldb = dev.put(B, dt)
    bc, pc, ldc = dev.put(C0, dt)
    dev.gemm(dt, 0, 0, 70, 50, 30, pa, lda, pb, ldb, -0.5, pc, ldc)
    dev.sync()
    want = A.astype(np.float64) @ B - 0.5 * C0
    assert rel_fro(dev.get(bc, (70, 50)), want) <= TIGHT[dt]


def test_degenerate_dimensions(dev):
    # k = 0 leaves beta * C; m = 0 / n = 0 are no-ops.
    C0 = np.arange(12, dtype=np.float32).reshape(3, 4, order="F")
    bc, pc, ldc = dev.put(C0, capi.F32)
    dev.gemm(capi.F32, 0, 0, 3, 4, 0, 0, 3, 0, 1, 1.0, pc, ldc)
    dev.gemm(capi.F32, 0, 0, 0, 4, 5, 0, 1, 0, 5, 0.0, pc, ldc)
    dev.gemm(capi.F32, 0, 0, 3, 0, 5, 0, 3, 0, 5, 0.0, pc, ldc)
    dev.sync()
    np.testing.assert_array_equal(dev.get(bc, (3, 4)), C0)
    dev.gemm(capi.F32, 0, 0, 3, 4, 0, 0, 3, 0, 1, 0.0, pc, ldc)
    dev.sync()
    np.testing.assert_array_equal(dev.get(bc, (3, 4)), np.zeros((3, 4)))


def test_argument_errors(dev):
    lib = dev.lib
    with pytest.raises(capi.GinnHipError, match="lda"):
        dev.gemm(capi.F32, 0, 0, 8, 8, 8, 16, 4, 16, 8, 0.0, 16, 8)
    with pytest.raises(capi.GinnHipError, match="dtype"):
        dev.gemm(7, 0, 0, 8, 8, 8, 16, 8, 16, 8, 0.0, 16, 8)
    with pytest.raises(capi.GinnHipError, match="NULL"):
        dev.gemm(capi.F32, 0, 0, 8, 8, 8, 0, 8, 16, 8, 0.0, 16, 8)
    assert "NULL" in lib.last_error()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("size", [512, 1024])
def test_square_full_check(dev, dt, op_a, op_b, size):
    run_case(dev, dt, op_a, op_b, size, size, size, 0.0, seed=size)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n", [1, 16, 64])
def test_skinny_full_check(dev, dt, n):
    # BASELINE config 2: M = K = 4096, N in {1, 16, 64}
    run_case(dev, dt, 0, 0, 4096, n, 4096, 0.0, seed=n)
    run_case(dev, dt, 1, 0, 4096, n, 4096, 1.0, seed=n + 1)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("size", [2048, 4096, 8192])
def test_square_large_sampled(dev, dt, op_a, op_b, size):
    """Full-size shapes: 64 seeded rows and 64 seeded columns of C checked in
    fp64, plus beta linearity (C1 - C0 == old C) on the whole matrix."""
    from gpu_util import TOL, TIGHT, stored
    torch = dev.torch
    from gpu_util import torch_dtype
    g = torch.Generator(device="cuda").manual_seed(size + 10 * dt)
    tdt = torch_dtype(dt)
    # Stored operands generated on the device (column-major == row-major of the transpose).
    a_rows, a_cols = (size, size)
    As = (torch.randn(a_cols, a_rows, generator=g, device="cuda") / np.sqrt(size)).to(tdt)
    Bs = torch.randn(a_cols, a_rows, generator=g, device="cuda").to(tdt)
    C = torch.empty(size, size, device="cuda", dtype=tdt)
    dev.gemm(dt, op_a, op_b, size, size, size, As.data_ptr(), size, Bs.data_ptr(), size, 0.0, C.data_ptr(), size)
    dev.sync()
    # Column-major stored X (ld = size) is X^T in torch's row-major view.
    A_st = As.float().cpu().numpy().T  # stored matrix
    B_st = Bs.float().cpu().numpy().T
    A = A_st.T if op_a else A_st      # logical m x k
    B = B_st.T if op_b else B_st      # logical k x n
    got = C.float().cpu().numpy().T
    rng = np.random.default_rng(size)
    rows = rng.choice(size, 64, replace=False)
    cols = rng.choice(size, 64, replace=False)
    want_rows = A[rows, :].astype(np.float64) @ B.astype(np.float64)
    want_cols = A.astype(np.float64) @ B[:, cols].astype(np.float64)
    e1, e2 = rel_fro(got[rows, :], want_rows), rel_fro(got[:, cols], want_cols)
    assert max(e1, e2) <= TOL[dt], (e1, e2)
    assert max(e1, e2) <= TIGHT[dt], (e1, e2)
    # beta linearity on the full matrix.
    C1 = torch.randn(size, size, generator=g, device="cuda").to(tdt)
    old = C1.clone()
    dev.gemm(dt, op_a, op_b, size, size, size, As.data_ptr(), size, Bs.data_ptr(), size, 1.0, C1.data_ptr(), size)
    dev.sync()
    diff = (C1.float() - C.float() - old.float()).norm() / old.float().norm()
    assert float(diff) <= TIGHT[dt] * 4


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k,batch", [(2, 5, 3, 4), (33, 17, 9, 5), (64, 64, 64, 3), (256, 256, 64, 8), (256, 64, 256, 8)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_strided_batched(dev, dt, op_a, op_b, m, n, k, batch, beta):
    """Batched product == per-slice product (the reference's own check,
    test/nodes.cu.cpp:1043-1115), strides = full slice sizes (ginn/prod.h:297-299)."""
    from gpu_util import TOL, TIGHT, round_to
    rng = np.random.default_rng(m + n + k + batch)
    a_shape = (k, m, batch) if op_a else (m, k, batch)
    b_shape = (n, k, batch) if op_b else (k, n, batch)
    A = round_to(rng.standard_normal(a_shape) / np.sqrt(k), dt)
    B = round_to(rng.standard_normal(b_shape), dt)
    C0 = round_to(rng.standard_normal((m, n, batch)), dt)
    ba, pa, _ = dev.put(A, dt)
    bb, pb, _ = dev.put(B, dt)
    bc, pc, _ = dev.put(C0, dt)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                 ctypes.c_void_p(pa), a_shape[0], a_shape[0] * a_shape[1],
                 ctypes.c_void_p(pb), b_shape[0], b_shape[0] * b_shape[1], beta,
                 ctypes.c_void_p(pc), m, m * n, batch)
    dev.sync()
    got = dev.get(bc, (m, n, batch))
    want = cgemm.bgemm(A, B, op_a, op_b, beta=beta, C=C0 if beta else None, kind="f64acc")
    err = rel_fro(got, want)
    assert err <= TOL[dt] and err <= TIGHT[dt], err


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m,n,k", [(4096, 1, 4096), (4096, 16, 4096), (1024, 1, 384), (640, 3, 100), (2048, 16, 70),
                                   (514, 7, 1030), (513, 2, 64), (8192, 9, 257), (4096, 64, 4096), (1000, 33, 300),
                                   (640, 40, 200), (515, 12, 129), (2052, 10, 1000), (4096, 13, 5000),
                                   (1024, 7, 600)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_skinny_shapes(dev, dt, m, n, k, beta):
    """Narrow right-hand sides (NN, tall A): the streaming kernel (up to 8
    columns for the 16-bit types, 16 for fp32), its matrix-core form (fp32,
    7 .. 16 columns, m a multiple of 4: ragged last row block, ragged K, K
    ranges longer than a block's B chunk) and the kernels that take over
    beyond, with and without K split over blocks, K not a multiple of
    anything, odd m (which only fp32 takes in the streaming kernel)."""
    run_case(dev, dt, 0, 0, m, n, k, beta, seed=m + n + k)


def test_skinny_matrix_core_long_k_range(dev):
    """fp32, 16 columns, so many row blocks that K is split in two: each half
    is longer than the B chunk a block holds, and the split count grows."""
    run_case(dev, capi.F32, 0, 0, 32768, 16, 2100, 1.0, seed=5)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("pad,offset", [(2, 0), (0, 2), (6, 4), (3, 1)])
def test_skinny_leading_dimension_and_alignment(dev, dt, pad, offset):
    """Padded leading dimensions and shifted base pointers; odd ones fall back
    to the generic kernel for the 16-bit types."""
    run_case(dev, dt, 0, 0, 1536, 5, 200, 1.0, pad=pad, offset=offset, seed=pad + offset)
    # 12 columns: the matrix-core form when the leading dimension and the base
    # keep 16-byte alignment (pad 0 or 4 with offset 0 or 4), the others otherwise
    run_case(dev, dt, 0, 0, 1536, 12, 600, 1.0, pad=pad, offset=offset, seed=pad + offset + 1)
    run_case(dev, dt, 0, 0, 1536, 12, 600, 0.0, pad=4, offset=offset, seed=pad + offset + 2)
