"""Parity of the tuned kernels against an fp64 product of the same rounded
inputs (fp16 / bf16: both kernels; fp32: the mid-size kernel).  The 256 x 256 x 64 kernel is taken for m, n multiples of
256, k a multiple of 64 and at least 256, and at least 144 tiles; the
128 x 128 x 64 kernel (optionally split-K) for the remaining shapes with m, n
multiples of 128 and k of 64.  Covered: every pipeline length with its own code
path, all four layouts, plain and accumulating epilogues, padded leading
dimensions, strided batches, split-K."""
import ctypes

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    from gpu_util import Dev
    d = Dev()
    yield d
    d.close()


def _operands(dev, dt, op_a, op_b, m, n, k, batch, seed):
    """Stored operands generated on the device; returns torch tensors whose
    row-major view is the transpose of the column-major stored matrix."""
    from gpu_util import torch_dtype
    torch = dev.torch
    g = torch.Generator(device="cuda").manual_seed(seed)
    a_rows, a_cols = (k, m) if op_a else (m, k)
    b_rows, b_cols = (n, k) if op_b else (k, n)
    A = (torch.randn(batch, a_cols, a_rows, generator=g, device="cuda") / np.sqrt(k)).to(torch_dtype(dt))
    B = torch.randn(batch, b_cols, b_rows, generator=g, device="cuda").to(torch_dtype(dt))
    return A, B, a_rows, b_rows


def _bound(dt):
    """Regression bound of a product with fp32 accumulation: the 16-bit types
    are dominated by the rounding of the result, fp32 by the length of K."""
    from gpu_util import TIGHT
    return 1e-5 if dt == capi.F32 else TIGHT[dt]


def _expected(A, B, op_a, op_b):
    # torch fp64 on the device: an independent library product of the same rounded inputs.
    As = A.double().transpose(1, 2)  # stored matrices, [batch, rows, cols]
    Bs = B.double().transpose(1, 2)
    Al = As.transpose(1, 2) if op_a else As
    Bl = Bs.transpose(1, 2) if op_b else Bs
    return Al @ Bl  # [batch, m, n]


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("k", [64, 128, 192, 256, 576])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_pipeline_lengths(dev, dt, op_a, op_b, k, beta):
    from gpu_util import TOL, TIGHT, torch_dtype
    torch = dev.torch
    m = n = 4096  # 256 tiles: k >= 256 runs the 256 x 256 kernel, shorter k the 128 x 128 one
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, k + 7 * dt)
    g = torch.Generator(device="cuda").manual_seed(99)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    if beta:
        want = want + beta * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
    dev.sync()
    got = C.double().transpose(1, 2)
    err = float((got - want).norm() / want.norm())
    assert err <= TOL[dt], err
    assert err <= TIGHT[dt], err


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k", [(3072, 3072, 320), (2304, 4096, 256), (3328, 2816, 384)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_fewest_tiles_of_the_large_kernel(dev, dt, op_a, op_b, m, n, k, beta):
    """144 tiles of 256 x 256 (the fewest the 256 x 256 kernel takes: 12 x 12 and 9 x 16) and 143
    (13 x 11, one short: the 128 x 128 kernel)."""
    from gpu_util import TIGHT, torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, m + n)
    g = torch.Generator(device="cuda").manual_seed(n)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    if beta:
        want = want + beta * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
    dev.sync()
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= TIGHT[dt], err


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
def test_rectangular_and_padded_ld(dev, dt, op_a, op_b):
    """m != n, leading dimensions larger than the row counts."""
    from gpu_util import TIGHT, torch_dtype
    torch = dev.torch
    m, n, k, pad = 3072, 4096, 320, 24
    g = torch.Generator(device="cuda").manual_seed(5)
    a_rows, a_cols = (k, m) if op_a else (m, k)
    b_rows, b_cols = (n, k) if op_b else (k, n)
    tdt = torch_dtype(dt)
    A = (torch.randn(a_cols, a_rows + pad, generator=g, device="cuda") / np.sqrt(k)).to(tdt)
    B = torch.randn(b_cols, b_rows + pad, generator=g, device="cuda").to(tdt)
    C = torch.full((n, m + pad), float("nan"), device="cuda", dtype=tdt)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), a_rows + pad, B.data_ptr(), b_rows + pad, 0.0,
             C.data_ptr(), m + pad)
    dev.sync()
    As, Bs = A[:, :a_rows].double().t(), B[:, :b_rows].double().t()
    want = (As.t() if op_a else As) @ (Bs.t() if op_b else Bs)
    got = C[:, :m].double().t()
    assert float((got - want).norm() / want.norm()) <= _bound(dt)
    assert bool(torch.isnan(C[:, m:].float()).all()), "padding rows of C were written"


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_strided_batch(dev, dt, op_a, op_b, beta):
    """The attention shape of the min-GPT configuration: 96 products of
    [512 x 512] * [512 x 64]-like tiles -> here 512 x 512 x 128, batch 16."""
    from gpu_util import TIGHT, torch_dtype
    torch = dev.torch
    m = n = 512
    k, batch = 128, 16
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, batch, 3)
    g = torch.Generator(device="cuda").manual_seed(4)
    C = torch.randn(batch, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    if beta:
        want = want + C.double().transpose(1, 2)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                 ctypes.c_void_p(A.data_ptr()), lda, A.shape[1] * A.shape[2],
                 ctypes.c_void_p(B.data_ptr()), ldb, B.shape[1] * B.shape[2], beta,
                 ctypes.c_void_p(C.data_ptr()), m, m * n, batch)
    dev.sync()
    got = C.double().transpose(1, 2)
    assert float((got - want).norm() / want.norm()) <= TIGHT[dt]


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
@pytest.mark.parametrize("m,n,k,batch", [(256, 256, 192, 6), (128, 384, 320, 3), (512, 512, 128, 2)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_strided_batch_of_few_tiles(dev, dt, op_a, op_b, m, n, k, batch, beta):
    """Batches whose slices together have few 128-wide tiles: the 64 x 64 tile shape of the mid-size
    kernel with a batch index (fp32: 96 .. 128 tiles of 64 x 64 without a K split)."""
    from gpu_util import torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, batch, 5 + batch)
    g = torch.Generator(device="cuda").manual_seed(k)
    C = torch.randn(batch, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    if beta:
        want = want + C.double().transpose(1, 2)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                 ctypes.c_void_p(A.data_ptr()), lda, A.shape[1] * A.shape[2],
                 ctypes.c_void_p(B.data_ptr()), ldb, B.shape[1] * B.shape[2], beta,
                 ctypes.c_void_p(C.data_ptr()), m, m * n, batch)
    dev.sync()
    got = C.double().transpose(1, 2)
    assert float((got - want).norm() / want.norm()) <= _bound(dt)


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(128, 128, 64), (384, 640, 192), (1024, 1024, 512), (2048, 2048, 128),
                                   (768, 768, 4096), (256, 128, 1024), (768, 4096, 768), (128, 256, 8192),
                                   (384, 64, 192), (64, 384, 320), (128, 64, 4096), (4096, 64, 4096),
                                   (64, 4096, 512), (128, 192, 64), (64, 128, 64),
                                   (4096, 16, 4096), (256, 100, 192), (128, 130, 64), (384, 37, 1024),
                                   (64, 200, 128), (1024, 1000, 256), (512, 512, 512), (192, 320, 256),
                                   (1024, 512, 128), (1024, 1024, 1024)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_mid_kernel_shapes(dev, dt, op_a, op_b, m, n, k, beta):
    """Shapes of the 128 x 128 kernel and its 128 x 64 / 64 x 128 / 64 x 64 variants (the last for
    outputs of few tiles: 512^3, 1024^3, 192 x 320, and with split K 128 x 64 x 4096): one
    tile, odd tile counts (no XCD grouping), one to many K tiles, and long-K /
    few-tile shapes that split K (the weight-gradient products of the GPT layer
    among them), and n that does not fill the last tile column (masked when B
    is K-contiguous, generic kernel otherwise)."""
    from gpu_util import TOL, TIGHT, torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, m + k + dt)
    g = torch.Generator(device="cuda").manual_seed(m)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    if beta:
        want = want + beta * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
    dev.sync()
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= _bound(dt), err


@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("k", [32, 64, 96, 128, 160, 288, 1056])
@pytest.mark.parametrize("m,n", [(256, 256), (128, 64), (64, 128), (512, 77)])
def test_mid_kernel_fp32_pipeline_lengths(dev, op_a, op_b, k, m, n):
    """fp32 through the mid-size kernel: a K tile is 32 values, so these K run
    one to 33 tiles (every prologue / steady-state / tail combination of the
    K loop), on all three tile shapes and with a masked last tile column."""
    torch = dev.torch
    dt = capi.F32
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, k + m)
    g = torch.Generator(device="cuda").manual_seed(k)
    C = torch.randn(1, n, m, generator=g, device="cuda")
    want = _expected(A, B, op_a, op_b) + 0.5 * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, 0.5, C.data_ptr(), m)
    dev.sync()
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= _bound(dt), err


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0)])
def test_mid_kernel_padded_ld(dev, dt, op_a, op_b):
    from gpu_util import TIGHT, torch_dtype
    torch = dev.torch
    m, n, k, pad = 384, 1152, 320, 40
    g = torch.Generator(device="cuda").manual_seed(6)
    a_rows, a_cols = (k, m) if op_a else (m, k)
    b_rows, b_cols = (n, k) if op_b else (k, n)
    tdt = torch_dtype(dt)
    A = (torch.randn(a_cols, a_rows + pad, generator=g, device="cuda") / np.sqrt(k)).to(tdt)
    B = torch.randn(b_cols, b_rows + pad, generator=g, device="cuda").to(tdt)
    C = torch.full((n, m + pad), float("nan"), device="cuda", dtype=tdt)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), a_rows + pad, B.data_ptr(), b_rows + pad, 0.0,
             C.data_ptr(), m + pad)
    dev.sync()
    As, Bs = A[:, :a_rows].double().t(), B[:, :b_rows].double().t()
    want = (As.t() if op_a else As) @ (Bs.t() if op_b else Bs)
    got = C[:, :m].double().t()
    assert float((got - want).norm() / want.norm()) <= _bound(dt)
    assert bool(torch.isnan(C[:, m:].float()).all()), "padding rows of C were written"


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k,batch", [(256, 256, 64, 128), (128, 128, 64, 264), (64, 64, 64, 1000),
                                         (256, 64, 256, 130), (64, 256, 256, 130), (64, 512, 512, 96),
                                         (512, 64, 512, 96), (192, 64, 128, 100), (64, 192, 192, 100),
                                         (1024, 64, 64, 40), (64, 128, 1024, 256)])
def test_small_slice_batches(dev, dt, op_a, op_b, m, n, k, batch):
    """The 4-wave kernel for batched products with small memory-bound slices (gemm_bsmall.hip): every
    layout, all four tile shapes (128 / 64 wide either way), one to sixteen K tiles (one and two LDS
    stages), batch counts that are and are not multiples of 8 (the XCD-aware order of the workgroups needs
    a multiple), against the fp64 product; NaN in C before the call must not survive (beta = 0)."""
    from gpu_util import torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, batch, 5)
    C = torch.full((batch, n, m), float("nan"), device="cuda", dtype=torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                 ctypes.c_void_p(A.data_ptr()), lda, A.shape[1] * A.shape[2],
                 ctypes.c_void_p(B.data_ptr()), ldb, B.shape[1] * B.shape[2], 0.0,
                 ctypes.c_void_p(C.data_ptr()), m, m * n, batch)
    dev.sync()
    got = C.double().transpose(1, 2)
    assert not bool(torch.isnan(got).any())
    assert float((got - want).norm() / want.norm()) <= _bound(dt)
    # slice by slice as well: a slice written to another one's place keeps the norm
    err = (got - want).flatten(1).norm(dim=1) / want.flatten(1).norm(dim=1)
    assert float(err.max()) <= _bound(dt) * 2


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("hs,nh,B,T", [(64, 12, 8, 512), (64, 3, 4, 128), (32, 5, 3, 72)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_two_level_batches_on_the_attention_layout(dev, dt, hs, nh, B, T, beta):
    """ginn_hip_gemm_strided_batched2 on operands as the projections of an attention layer leave them: K, Q, V
    are [hs nh x B T] matrices (element (e, h, b, t) at e + hs (h + nh (b + B t))), slice z = b + B h of each is
    the [hs x T] matrix with leading dimension hs nh B at 64 h + hs nh b -- two levels of strides.  Scores
    S = K^T Q (TN, [T x T] slices, contiguous), output Y = V P written back into the [hs nh x B T] layout, and
    the gradient dK^T = Q dS^T (NT) written strided as well.  16-bit 64-row slices take the small-slice kernel in
    one launch; fp32 and the odd sizes run level by level on the other kernels; against numpy fp64."""
    from gpu_util import round_to, torch_dtype
    torch = dev.torch
    rng = np.random.default_rng(hs + nh + B + T)
    C_ = hs * nh

    def proj():
        return round_to(rng.standard_normal((hs, nh, B, T)) / np.sqrt(hs), dt)

    K, Q, V = proj(), proj(), proj()
    up = lambda a: torch.from_numpy(np.ascontiguousarray(a.reshape(-1, order="F"))).to("cuda").to(torch_dtype(dt))
    dK_, dQ_, dV_ = up(K), up(Q), up(V)
    ld, s_b, s_h, batch = C_ * B, C_, hs, B * nh
    call = lambda *a: dev.lib.call("ginn_hip_gemm_strided_batched2", dev.ctx, dt, *a)
    ptr = lambda t: ctypes.c_void_p(t.data_ptr())
    # scores: [T x T] per slice, contiguous slices numbered z = b + B h
    S0 = round_to(rng.standard_normal((T, T, B, nh)), dt)
    dS = up(S0)
    call(1, 0, T, T, hs, ptr(dK_), ld, s_b, s_h, ptr(dQ_), ld, s_b, s_h, beta, ptr(dS), T, T * T, T * T * B, B, nh)
    dev.sync()
    got = dS.double().cpu().numpy().reshape((T, T, B, nh), order="F")
    want = np.einsum("ehbt,ehbu->tubh", K.astype(np.float64), Q.astype(np.float64)) + beta * S0
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= _bound(dt)
    # output: Y[e, h, b, t] = sum_u V[e, h, b, u] P[u, t, b, h], written in the projections' layout
    P = round_to(rng.uniform(0, 2.0 / T, (T, T, B, nh)), dt)
    Y0 = proj()
    dP, dY = up(P), up(Y0)
    call(0, 0, hs, T, T, ptr(dV_), ld, s_b, s_h, ptr(dP), T, T * T, T * T * B, beta, ptr(dY), ld, s_b, s_h, B, nh)
    dev.sync()
    got = dY.double().cpu().numpy().reshape((hs, nh, B, T), order="F")
    want = np.einsum("ehbu,utbh->ehbt", V.astype(np.float64), P.astype(np.float64)) + beta * Y0
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= _bound(dt)
    # gradient of K through its transposed view: dKview[e, h, b, t] = sum_u Q[e, h, b, u] G[t, u, b, h]
    G = round_to(rng.standard_normal((T, T, B, nh)) / np.sqrt(T), dt)
    D0 = proj()
    dG, dD = up(G), up(D0)
    call(0, 1, hs, T, T, ptr(dQ_), ld, s_b, s_h, ptr(dG), T, T * T, T * T * B, beta, ptr(dD), ld, s_b, s_h, B, nh)
    dev.sync()
    got = dD.double().cpu().numpy().reshape((hs, nh, B, T), order="F")
    want = np.einsum("ehbu,tubh->ehbt", Q.astype(np.float64), G.astype(np.float64)) + beta * D0
    assert np.linalg.norm(got - want) / np.linalg.norm(want) <= _bound(dt)


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("op_a,op_b,m,n,k", [(0, 0, 512, 512, 64), (0, 0, 256, 256, 64), (0, 1, 256, 256, 64),
                                             (1, 0, 256, 128, 256), (0, 0, 128, 512, 512), (0, 0, 256, 64, 256),
                                             (0, 1, 256, 64, 256), (1, 0, 64, 256, 256), (0, 0, 64, 512, 512),
                                             (0, 1, 64, 512, 512), (1, 0, 512, 64, 512)])
def test_mid_kernel_attention_batches(dev, dt, op_a, op_b, m, n, k):
    """Strided batches with the shapes of the attention products."""
    from gpu_util import TIGHT, torch_dtype
    torch = dev.torch
    batch = 24
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, batch, 11)
    C = torch.zeros(batch, n, m, device="cuda", dtype=torch_dtype(dt))
    want = _expected(A, B, op_a, op_b)
    dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                 ctypes.c_void_p(A.data_ptr()), lda, A.shape[1] * A.shape[2],
                 ctypes.c_void_p(B.data_ptr()), ldb, B.shape[1] * B.shape[2], 0.0,
                 ctypes.c_void_p(C.data_ptr()), m, m * n, batch)
    dev.sync()
    got = C.double().transpose(1, 2)
    assert float((got - want).norm() / want.norm()) <= _bound(dt)


@pytest.mark.parametrize("seed", [1, 2, 3, 4])
def test_seeded_random_shapes(dev, seed):
    """Which kernel takes a product is decided by its extents, type, layout and batch (tile counts against
    the number of CUs, K against the split limits): 250 seeded draws per case from extents on both sides of
    every such limit, aligned and ragged, all four layouts, beta 0 / 0.5 / 1, some as strided batches, each
    against the fp64 product of the same rounded operands."""
    import random
    from gpu_util import torch_dtype
    torch = dev.torch
    rng = random.Random(seed)
    ms = [64, 128, 192, 256, 320, 384, 512, 640, 768, 1024, 1280, 1536, 2048, 2304, 3072, 4096, 100, 200, 1000, 33,
          72, 136, 264, 520, 1032, 2056, 3080]
    ns = ms + [1, 4, 8, 9, 16, 37, 40, 72, 130, 504]
    ks = [32, 64, 96, 128, 192, 256, 320, 512, 768, 1024, 1056, 1536, 2048, 2052, 3072, 4096, 100, 1000,
          72, 264, 328, 520, 4104]
    worst = {}
    for it in range(250):
        dt = rng.choice([capi.F32, capi.F16, capi.BF16])
        m, n, k = rng.choice(ms), rng.choice(ns), rng.choice(ks)
        op_a, op_b = rng.choice([(0, 0), (0, 1), (1, 0), (1, 1)])
        beta = rng.choice([0.0, 1.0, 0.5])
        if m * n * k > 3e10 or m * n > 2 ** 24:
            continue
        batch = rng.choice([1, 1, 1, 2, 5]) if m * n * k < 2e9 else 1
        A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, batch, 1000 * seed + it)
        g = torch.Generator(device="cuda").manual_seed(it)
        C = torch.randn(batch, n, m, generator=g, device="cuda").to(torch_dtype(dt))
        want = _expected(A, B, op_a, op_b) + beta * C.double().transpose(1, 2)
        if batch == 1:
            dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
        else:
            dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k,
                         ctypes.c_void_p(A.data_ptr()), lda, A.shape[1] * A.shape[2],
                         ctypes.c_void_p(B.data_ptr()), ldb, B.shape[1] * B.shape[2], beta,
                         ctypes.c_void_p(C.data_ptr()), m, m * n, batch)
        dev.sync()
        err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
        assert err <= 2 * _bound(dt), (dt, op_a, op_b, m, n, k, batch, beta, err)
        worst[dt] = max(worst.get(dt, 0.0), err)
    assert len(worst) == 3


@pytest.mark.parametrize("dt", [capi.F32, capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(1024, 1024, 1000), (2000, 2000, 2000), (1000, 1024, 1024), (1160, 1096, 1032),
                                   (1024, 520, 4100),
                                   # multiples of 128 but not of 256: 256 x 256 kernel for the core, strips beside it
                                   (3200, 3200, 320), (3328, 4224, 256)])
@pytest.mark.parametrize("beta", [0.0, 1.0])
def test_ragged_extents_with_aligned_leading_dimensions(dev, dt, op_a, op_b, m, n, k, beta):
    """Extents that are no multiples of the tuned kernels' tiles while leading dimensions and pointers
    allow 16-byte accesses: the product is cut into the last K % 64 (32 for fp32) values over the whole
    output, the aligned core on the tuned kernels, and the ragged rows / columns around it (16-bit extents
    that are multiples of 128 but not of 256: a core of 256-multiples and strips of 128)."""
    from gpu_util import torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, m + n + k)
    g = torch.Generator(device="cuda").manual_seed(k)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b) + beta * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
    dev.sync()
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= 2 * _bound(dt), err


@pytest.mark.parametrize("dt", [capi.F32, capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(1501, 1503, 1505), (1024, 1024, 1001), (1001, 1024, 1024), (2047, 2049, 515)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_odd_leading_dimensions_of_large_products(dev, dt, op_a, op_b, m, n, k, beta):
    """Leading dimensions that rule out 16-byte accesses (odd row counts): a large product runs on copies
    with padded leading dimensions from the context's pool (one, two or all three of A, B, C copied; C
    copied in when beta reads it and always copied back), a smaller one on the any-shape kernel."""
    from gpu_util import torch_dtype
    torch = dev.torch
    A, B, lda, ldb = _operands(dev, dt, op_a, op_b, m, n, k, 1, m + 2 * n + 3 * k)
    g = torch.Generator(device="cuda").manual_seed(m)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, op_a, op_b) + beta * C.double().transpose(1, 2)
    dev.gemm(dt, op_a, op_b, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, beta, C.data_ptr(), m)
    dev.sync()
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= 2 * _bound(dt), err


@pytest.mark.parametrize("dt", [capi.F16, capi.F32])
@pytest.mark.parametrize("budget", [0, 1 << 20, None])
def test_products_on_copies_keep_within_the_budget_for_temporaries(dev, dt, budget):
    """A product on operands with odd leading dimensions may take device memory for padded copies
    (ginn_hip_gemm_temp_budget; cuBLAS computes in place, ginn/prod.h:46-62).  With a budget of 0, or one
    the copies do not fit, it runs in place on the any-shape kernel instead: same result, nothing taken
    from the context's pool; with the default budget the copies are made and returned to the pool."""
    from ctypes import byref, c_size_t
    from gpu_util import torch_dtype
    torch = dev.torch
    m, n, k = 1501, 1503, 1505
    A, B, lda, ldb = _operands(dev, dt, 0, 0, m, n, k, 1, 77)
    g = torch.Generator(device="cuda").manual_seed(3)
    C = torch.randn(1, n, m, generator=g, device="cuda").to(torch_dtype(dt))
    want = _expected(A, B, 0, 0) + 0.5 * C.double().transpose(1, 2)

    def blocks():
        cached, count = c_size_t(0), c_size_t(0)
        dev.lib.call("ginn_hip_pool_stats", dev.ctx, byref(cached), byref(count))
        return count.value

    dev.lib.call("ginn_hip_pool_trim", dev.ctx)
    before = blocks()
    try:
        if budget is not None:
            dev.lib.call("ginn_hip_gemm_temp_budget", dev.ctx, budget)
        dev.gemm(dt, 0, 0, m, n, k, A.data_ptr(), lda, B.data_ptr(), ldb, 0.5, C.data_ptr(), m)
        dev.sync()
    finally:
        dev.lib.call("ginn_hip_gemm_temp_budget", dev.ctx, 2 << 30)
    took = blocks() - before
    assert (took == 0) if budget is not None else (took >= 3), took
    err = float((C.double().transpose(1, 2) - want).norm() / want.norm())
    assert err <= 2 * _bound(dt), err


def _masked_case(dev, dt, op_a, op_b, m, n, k, beta, batch=1):
    """One product whose operands and result sit in buffers with 8 NaN-filled rows of padding below every
    column (leading dimensions stay multiples of 8): a tile edge that reads beyond an extent shows up as
    NaN in the result, and one that stores beyond it as a changed padding row."""
    from gpu_util import round_to
    rng = np.random.default_rng(m + 3 * n + 7 * k + op_a + 2 * op_b)
    a_shape = (k, m) if op_a else (m, k)
    b_shape = (n, k) if op_b else (k, n)
    pad = 8
    hs, bufs = [], []
    for shape, scale in ((a_shape, 1 / np.sqrt(k)), (b_shape, 1.0), ((m, n), 1.0)):
        h = round_to(rng.standard_normal(shape + (batch,)) * scale, dt)
        hs.append(h)
        bufs.append(dev.put(h.reshape(shape[0], -1, order="F"), dt, pad_rows=pad))
    (A, B, C), ((ba, pa, lda), (bb, pb, ldb), (bc, pc, ldc)) = hs, bufs
    es = 4 if dt == capi.F32 else 2
    if batch == 1:
        dev.gemm(dt, op_a, op_b, m, n, k, pa, lda, pb, ldb, beta, pc, ldc)
    else:
        dev.lib.call("ginn_hip_gemm_strided_batched", dev.ctx, dt, op_a, op_b, m, n, k, ctypes.c_void_p(pa), lda,
                     lda * a_shape[1], ctypes.c_void_p(pb), ldb, ldb * b_shape[1], beta, ctypes.c_void_p(pc), ldc,
                     ldc * n, batch)
    dev.sync()
    whole = bc.to(dev.torch.float32).cpu().numpy().reshape(batch * n, ldc)
    assert np.isnan(whole[:, m:]).all(), "rows below the result were written"
    got = whole[:, :m].reshape(batch, n, m).transpose(2, 1, 0)
    assert not np.isnan(got).any(), "padding of an operand (or K beyond its end) reached the result"
    for z in range(batch):
        a64, b64 = A[..., z].astype(np.float64), B[..., z].astype(np.float64)
        want = (a64.T if op_a else a64) @ (b64.T if op_b else b64) + beta * C[..., z].astype(np.float64)
        err = np.linalg.norm(got[..., z] - want) / np.linalg.norm(want)
        assert err <= 2 * _bound(dt), (z, err)
    del es


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(136, 200, 72), (264, 72, 136), (520, 328, 1000), (1000, 1000, 1000),
                                   (72, 1032, 264), (1288, 520, 96), (200, 2056, 3000)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_masked_tile_edges_of_the_128_wide_kernels(dev, dt, op_a, op_b, m, n, k, beta):
    """Extents that are multiples of 8 but not of the tiles, leading dimensions that allow 16-byte accesses:
    the last tile row, tile column and K tile are masked inside the tuned kernels (clamped loads, zeros
    beyond K, masked stores) in every layout, as cuBLAS takes any m, n, k (ginn/prod.h:46-62).  The last
    shape runs with K split over workgroups."""
    _masked_case(dev, dt, op_a, op_b, m, n, k, beta)


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b", [(0, 0), (0, 1), (1, 0), (1, 1)])
@pytest.mark.parametrize("m,n,k", [(3080, 3208, 264), (3848, 3976, 328), (4000, 4000, 1000)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_masked_tile_edges_of_the_256_wide_kernel(dev, dt, op_a, op_b, m, n, k, beta):
    """The same on the 256 x 256 kernel (at least 144 tiles), plain and accumulating epilogue; the shapes
    of the reference's own benchmark are 4000^3, 1000^3 and 16000 x 4000 (examples/bench.cu.cpp:216-220)."""
    _masked_case(dev, dt, op_a, op_b, m, n, k, beta)


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("op_a,op_b,m,n,k", [(0, 0, 504, 504, 64), (0, 1, 504, 64, 504), (1, 0, 64, 504, 504),
                                             (0, 0, 64, 504, 504), (0, 1, 64, 504, 504), (1, 0, 504, 504, 64),
                                             (0, 0, 200, 64, 136), (1, 1, 72, 1000, 64)])
def test_masked_tile_edges_of_the_small_slice_kernel(dev, dt, op_a, op_b, m, n, k):
    """Attention products with a sequence length that is no multiple of 64 (T = 504, head size 64, 96
    slices): forward and both gradients of Q K^T and P V, each slice's last tiles masked."""
    _masked_case(dev, dt, op_a, op_b, m, n, k, 0.0, batch=96 if max(m, n, k) <= 504 else 40)


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16, capi.F32])
@pytest.mark.parametrize("n", [1, 2, 3, 5, 8, 9, 12, 13, 16])
@pytest.mark.parametrize("m,k", [(2048, 1024), (4096, 4096), (2056, 1040), (4104, 2064), (2048, 8208), (4096, 1040),
                                 (4104, 1056)])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_narrow_right_hand_sides_in_one_launch(dev, dt, n, m, k, beta):
    """NN products with at most 16 columns over a tall A of up to 24 MiB (fp32: 8 .. 16 columns, up to 32 MiB)
    run as one launch of 16-row strips over all of K (gemm_strip.hip; the degenerate end of
    ginn/prod.h:32-66), larger ones on the kernels that split K over workgroups: every width of the B
    loads (n <= 4, 8, 16), a last strip that is partly filled, K ranges that split unevenly over the four
    waves and buffers that are partly used, plain and accumulating epilogue, NaN padding around every operand."""
    _masked_case(dev, dt, 0, 0, m, n, k, beta)
