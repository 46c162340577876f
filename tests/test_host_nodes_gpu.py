"""The header-only C++ host layer (ginn_amd/ginn: Tensor, Graph, ProdNode,
BatchedProdNode, AffineNode, nonlinearity nodes) on the HIP device, compared
with the numpy node oracle.  Protocol of test/check_node.h:27-121 and
test/testutil.h:93-171: the expression is evaluated as e = f() + f() and the
loss is Sum(mask * e), so every input gradient accumulates over two paths."""
import ctypes
from pathlib import Path

import numpy as np
import pytest

from conftest import farr, rel_fro
from ginn_amd import capi
from oracle import nodes as N

pytestmark = pytest.mark.gpu

DTYPES = [capi.F32, capi.F16, capi.BF16]
SHIM = Path(__file__).resolve().parent / "cpp" / "libhost_shim.so"


@pytest.fixture(scope="module")
def shim():
    if not SHIM.exists():
        pytest.fail(f"{SHIM} is missing: run __graft_entry__.build()")
    capi.load()  # resolves libginn_hip.so first
    lib = ctypes.CDLL(str(SHIM))
    lib.shim_last_error.restype = ctypes.c_char_p
    lib.shim_expect_throw.restype = ctypes.c_char_p
    return lib


def fptr(a):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def dims(shape):
    return (ctypes.c_long * max(1, len(shape)))(*shape)


def f32(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float32))


def check(lib, rc):
    assert rc == 0, lib.shim_last_error().decode()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("a_shape,b_shape,batched", [
    ((2, 3), (3, 2), 0), ((64, 48), (48, 33), 0), ((130, 70), (70, 96), 0), ((4, 6, 5), (30, 7), 0),
    ((2, 3, 4), (3, 5, 4), 1), ((2, 3, 2, 2), (3, 5, 2, 2), 1), ((64, 32, 8), (32, 48, 8), 1)])
def test_prod_nodes(shim, dt, a_shape, b_shape, batched):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(len(a_shape) * 100 + a_shape[0])
    a = round_to(rng.uniform(-1, 1, a_shape), dt)
    b = round_to(rng.uniform(-1, 1, b_shape), dt)
    fwd = N.batched_prod_forward if batched else N.prod_forward
    bwd = N.batched_prod_backward if batched else N.prod_backward
    want_f = fwd(a.astype(np.float64), b.astype(np.float64))
    mask = round_to(rng.uniform(-1, 1, want_f.shape), dt)
    out = np.zeros(want_f.shape, np.float32, order="F")
    da = np.zeros(a_shape, np.float32, order="F")
    db = np.zeros(b_shape, np.float32, order="F")
    check(shim, shim.shim_prod_node(dt, batched, dims(a_shape), len(a_shape), dims(b_shape), len(b_shape),
                                    fptr(f32(a)), fptr(f32(b)), fptr(f32(mask)), fptr(out), fptr(da), fptr(db)))
    want_da, want_db = bwd(a.astype(np.float64), b.astype(np.float64), mask.astype(np.float64))
    # e = f + f: values double; with 16-bit storage each f is rounded before the sum.
    assert rel_fro(out, 2 * want_f) <= TOL[dt]
    assert rel_fro(da, 2 * want_da) <= TOL[dt] * 2
    assert rel_fro(db, 2 * want_db) <= TOL[dt] * 2


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("product", ["QK^T", "PV"])
def test_attention_products_through_batched_prod_node(shim, dt, product):
    """The attention configuration at its stated size: batch * heads = 128 slices,
    QK^T = [256 x 64] * [64 x 256] and P V = [256 x 256] * [256 x 64] with Q, K,
    V ~ N(0, 1) and P the row-softmax of a seeded N(0, 1) matrix, 16-bit storage,
    through BatchedProdNode (ginn/node/prod.h:93-169): value and both input
    gradients (dA = dY B^T per slice, dB = A^T dY per slice) against the fp64
    oracle, protocol of test/nodes.cu.cpp:1043-1115 (e = f() + f(), masked sum)."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(4 if product == "PV" else 44)
    batch = 128
    if product == "QK^T":
        a_shape, b_shape = (256, 64, batch), (64, 256, batch)
        a = rng.standard_normal(a_shape)
        b = rng.standard_normal(b_shape)
    else:
        a_shape, b_shape = (256, 256, batch), (256, 64, batch)
        s = rng.standard_normal(a_shape)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        a = e / e.sum(axis=1, keepdims=True)  # every row of every slice sums to 1
        b = rng.standard_normal(b_shape)
    a, b = round_to(a, dt), round_to(b, dt)
    a64, b64 = a.astype(np.float64), b.astype(np.float64)
    want_f = N.batched_prod_forward(a64, b64)
    mask = round_to(rng.uniform(-1, 1, want_f.shape), dt)
    out = np.zeros(want_f.shape, np.float32, order="F")
    da = np.zeros(a_shape, np.float32, order="F")
    db = np.zeros(b_shape, np.float32, order="F")
    check(shim, shim.shim_prod_node(dt, 1, dims(a_shape), 3, dims(b_shape), 3, fptr(f32(a)), fptr(f32(b)),
                                    fptr(f32(mask)), fptr(out), fptr(da), fptr(db)))
    want_da, want_db = N.batched_prod_backward(a64, b64, mask.astype(np.float64))
    assert rel_fro(out, 2 * want_f) <= TOL[dt]
    assert rel_fro(da, 2 * want_da) <= TOL[dt]
    assert rel_fro(db, 2 * want_db) <= TOL[dt]
    # independent of the oracle: slice 77 of the value is the plain product of slice 77
    np.testing.assert_allclose(out[:, :, 77] / 2, a64[:, :, 77] @ b64[:, :, 77], rtol=0, atol=TOL[dt] * np.abs(want_f).max())


@pytest.mark.parametrize("dt", DTYPES)
def test_prod_reference_golden(shim, golden, dt):
    g = golden["prod"]
    W, V = farr(g["W"], np.float32), farr(g["V"], np.float32)
    out = np.zeros((2, 2), np.float32, order="F")
    mask = np.ones((2, 2), np.float32, order="F")
    da = np.zeros((2, 3), np.float32, order="F")
    db = np.zeros((3, 2), np.float32, order="F")
    check(shim, shim.shim_prod_node(dt, 0, dims((2, 3)), 2, dims((3, 2)), 2, fptr(W), fptr(V), fptr(mask),
                                    fptr(out), fptr(da), fptr(db)))
    eps = {capi.F32: 1e-6, capi.F16: 1e-2, capi.BF16: 3e-2}[dt]
    np.testing.assert_allclose(out / 2, farr(g["WV"], np.float32), rtol=eps)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("act", [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.SOFTMAX, N.GELU, N.GELU2])
@pytest.mark.parametrize("case", ["vector", "broadcast", "high_rank", "two_pairs", "mlp_layer", "fixed_input"])
def test_affine_node(shim, dt, act, case):
    """The Affine cases of test/nodes.cu.cpp:1117-1200 (vector, column
    broadcast, rank-3 right-hand side, all epilogues) plus two pairs, a layer
    of the MLP configuration, and an input without gradient."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(act * 10 + len(case))
    has_grad = None
    if case == "vector":
        shapes = [(2, 3), (3, 1), (2, 1)]
    elif case == "broadcast":
        shapes = [(2, 3), (3, 2), (2, 1)]
    elif case == "high_rank":
        shapes = [(2, 3), (3, 2, 2), (2,)]
    elif case == "two_pairs":
        shapes = [(24, 16), (16, 9), (24, 40), (40, 9), (24,)]
    elif case == "mlp_layer":
        shapes = [(512, 784), (784, 64), (512,)]
    else:
        shapes = [(20, 12), (12, 7), (20,)]
        has_grad = [1, 0, 1]
    has_grad = has_grad or [1] * len(shapes)
    ins = []
    for i, s in enumerate(shapes):
        scale = 1.0 / np.sqrt(s[1]) if (i % 2 == 0 and i + 1 < len(shapes)) else 1.0
        x = rng.uniform(-1, 1, s) * scale
        if act == N.RELU and i == 0:
            x = x * 10  # as the reference: keep pre-activations away from the kink
        ins.append(round_to(x, dt))
    ins64 = [x.astype(np.float64) for x in ins]
    want_v, want_pre = N.affine_forward(act, ins64)
    mask = round_to(rng.uniform(-1, 1, want_v.shape), dt)
    want_g = N.affine_backward(act, ins64, want_v, want_pre, mask.astype(np.float64))
    out = np.zeros(want_v.shape, np.float32, order="F")
    grads = [np.zeros(s, np.float32, order="F") for s in shapes]
    flat_dims = [d for s in shapes for d in s]
    n = len(shapes)
    check(shim, shim.shim_affine_node(
        dt, act, n, (ctypes.c_long * len(flat_dims))(*flat_dims), (ctypes.c_int * n)(*[len(s) for s in shapes]),
        (ctypes.POINTER(ctypes.c_float) * n)(*[fptr(f32(x)) for x in ins]), (ctypes.c_int * n)(*has_grad),
        fptr(f32(mask)), fptr(out), (ctypes.POINTER(ctypes.c_float) * n)(*[fptr(g) for g in grads])))
    tol = TOL[dt] * (2 if dt != capi.F32 else 1)
    assert rel_fro(out, 2 * want_v) <= tol
    for i in range(n):
        if has_grad[i]:
            assert rel_fro(grads[i], 2 * want_g[i]) <= 3 * tol, (case, i)
        else:
            assert not grads[i].any()


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("act", [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.SOFTMAX, N.GELU, N.GELU2, N.LOG, N.SQRT])
def test_nonlin_nodes(shim, dt, act):
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(act)
    shape = (6, 5)
    x = rng.uniform(-1, 1, shape)
    if act in (N.LOG, N.SQRT):
        x = np.abs(x) + 0.5
    x = round_to(x, dt)
    want = N.nonlin_forward(act, x.astype(np.float64))
    mask = round_to(rng.uniform(-1, 1, shape), dt)
    out = np.zeros(shape, np.float32, order="F")
    dx = np.zeros(shape, np.float32, order="F")
    check(shim, shim.shim_nonlin_node(dt, act, dims(shape), 2, fptr(f32(x)), fptr(f32(mask)), fptr(out), fptr(dx)))
    want_dx = N.nonlin_backward(act, mask.astype(np.float64), x.astype(np.float64), want)
    assert rel_fro(out, 2 * want) <= TOL[dt] * 2
    assert rel_fro(dx, 2 * want_dx) <= TOL[dt] * 4


@pytest.mark.parametrize("case", ["tensor_ctors", "tensor_ops", "forwardedness", "gradfulness", "arena_tensors",
                                  "arena_nodes", "arena_limits", "layout_goldens",
                                  "arithmetic_goldens", "select_goldens"])
def test_reference_structural_cases(shim, case):
    """The reference's structural tests on the HIP device: Tensor construction /
    copy / move / assignment across devices, resize, set, serialize and errors
    (test/tensor.cu.cpp), forwardedness and gradient allocation rules
    (test/graph.cpp:26-115), the byte accounting of the preallocated device
    arena for tensors and nodes (test/dev.cu.cpp:122-178), and the known answers of
    the layout nodes (Stack, Cat, RowwiseCat / RowwiseUncat, Reshape, RankView, Slice,
    Chip: test/nodes.cu.cpp:66-306) and of the arithmetic nodes (test/nodes.cu.cpp:443-656), both for Real, Half,
    BFloat16 and Int."""
    shim.shim_structural.restype = ctypes.c_char_p
    report = shim.shim_structural(case.encode()).decode()
    assert report == "", report


@pytest.mark.parametrize("dt,shape0,shape1", [
    (capi.F32, (512, 64, 784), (10, 64, 512)),       # generic kernel, split-K partials in the workspace
    (capi.F32, (4096, 1, 4096), (4096, 16, 4096)),   # skinny kernels, K split over blocks
    (capi.BF16, (768, 768, 4096), (4096, 1, 4096)),  # 128 x 128 family with split-K, and the 16-bit skinny kernel
])
def test_one_context_two_host_threads(shim, dt, shape0, shape1):
    """Two host threads enqueue split-K products on the same context at the same
    time; each keeps its partial sums in the context's one workspace.  Every
    iteration accumulates into C, so one interleaved fold would show."""
    from gpu_util import TOL, round_to
    rng = np.random.default_rng(shape0[0] + shape1[1])
    iters = 16
    ops, outs = [], []
    for m, n, k in (shape0, shape1):
        a = round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt)
        b = round_to(rng.standard_normal((k, n)), dt)
        ops.append((a, b))
        outs.append(np.zeros((m, n), np.float32, order="F"))
    args = []
    for (a, b), (m, n, k), c in zip(ops, (shape0, shape1), outs):
        args += [(ctypes.c_long * 3)(m, n, k), fptr(f32(a)), fptr(f32(b)), fptr(c)]
    check(shim, shim.shim_two_threads(dt, iters, *args))
    for (a, b), c in zip(ops, outs):
        want = iters * (a.astype(np.float64) @ b.astype(np.float64))
        assert rel_fro(c, want) <= TOL[dt]


def test_error_paths(shim):
    """Failure handling of the host layer (ginn/prod.h:236-238,
    ginn/node/prod.h:95-101, ginn/node/affine.h:148-149, ginn/dev.h:238-241,
    ginn/tensor.h:328-329): exceptions, never a wrong result or a fault."""
    expect = {0: "a_inner == b_inner", 1: "at least rank 3", 2: "% 2", 3: "out of memory", 4: "Cpu tensors",
              5: "HIP device only"}
    for which, text in expect.items():
        msg = shim.shim_expect_throw(which).decode()
        assert text in msg, (which, msg)


@pytest.mark.parametrize("frozen", [0, 1])
@pytest.mark.parametrize("rows,cols1,cols2", [(8, 3, 5), (64, 16, 16), (33, 7, 2), (256, 64, 1)])
def test_level_executor_replans(shim, rows, cols1, cols2, frozen):
    """The executor's launch plans follow the graph: after an input changes its
    shape (or only its storage) the next pass rebuilds them, and values and
    gradients are those of node-by-node execution and of the oracle."""
    rng = np.random.default_rng(rows * 100 + cols2)
    x1 = f32(rng.standard_normal((rows, cols1)))
    x2 = f32(rng.standard_normal((rows, cols2)))
    outs = [np.zeros((rows, cols2), np.float32, order="F") for _ in range(4)]
    rebuilt = ctypes.c_int(-1)
    check(shim, shim.shim_executor_replan(rows, cols1, cols2, fptr(x1), fptr(x2), frozen, *map(fptr, outs),
                                          ctypes.byref(rebuilt)))
    y_exec, dx_exec, y_plain, dx_plain = outs
    if cols1 != cols2:
        assert rebuilt.value > 0  # other sizes, other storage: the old plans cannot be replayed
    np.testing.assert_array_equal(y_exec, y_plain)
    assert rel_fro(dx_exec, dx_plain) <= 1e-6
    x = x2.astype(np.float64)
    sig = 1.0 / (1.0 + np.exp(-x))
    y = np.tanh(x) * sig + x + np.maximum(x, 0)
    dy = 2 * y
    dx = dy * ((1 - np.tanh(x) ** 2) * sig + np.tanh(x) * sig * (1 - sig) + 1 + (x > 0))
    assert rel_fro(y_exec, y) <= 1e-5
    assert rel_fro(dx_exec, dx) <= 1e-4


@pytest.mark.parametrize("rows,cols,hidden", [(16, 8, 32), (784, 64, 512), (5, 3, 7)])
def test_level_executor_recorded_pass(shim, rows, cols, hidden):
    """A frozen pass recorded as a device graph: replayed several times, with new
    input values uploaded between the replays, every replay gives exactly what
    the same pass gives launch by launch."""
    rng = np.random.default_rng(rows + hidden)
    replays = 4
    w = f32(rng.standard_normal((hidden, rows)) / np.sqrt(rows))
    b = f32(rng.standard_normal(hidden))
    xs = f32(rng.standard_normal((rows * cols, replays)))
    worst = ctypes.c_float(-1)
    check(shim, shim.shim_executor_graph(rows, cols, hidden, replays, fptr(w), fptr(b), fptr(xs),
                                         ctypes.byref(worst)))
    assert worst.value == 0.0
