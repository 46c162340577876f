"""Whole graphs of the build target's configurations, built with the C++ host
layer (ginn_amd/examples/configs.cpp) on the HIP device and compared with the
CPU oracle: the MLP of AffineNodes, the reference's Autobatch equivalence
cases (test/autobatch.cpp:72-190) and the autobatched LSTM gates."""
import ctypes
from pathlib import Path

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi
from oracle import nodes as N

pytestmark = pytest.mark.gpu

SHIM = capi.LIB_PATH.parent / "libginn_examples.so"
FP = ctypes.POINTER(ctypes.c_float)


@pytest.fixture(scope="module")
def shim():
    if not SHIM.exists():
        pytest.fail(f"{SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(SHIM))
    lib.scenario_last_error.restype = ctypes.c_char_p
    lib.scenario_timed_fills.restype = ctypes.c_long
    lib.scenario_late_sum_columns.restype = ctypes.c_long
    return lib


def fptr(a):
    return a.ctypes.data_as(FP)


def f32(a):
    return np.asfortranarray(np.asarray(a, dtype=np.float32))


def ptrs(arrays):
    return (FP * len(arrays))(*[fptr(a) for a in arrays])


def check(lib, rc):
    assert rc == 0, lib.scenario_last_error().decode()


def xavier(rng, rows, cols):
    """U[-a, a], a = sqrt(6 / (0.5 (rows + cols)))  (ginn/init/init.h:45-51)."""
    a = np.sqrt(6.0 / (0.5 * (rows + cols)))
    return rng.uniform(-a, a, (rows, cols))


# ---------------------------------------------------------------------------
# MLP: batch 64, 784 -> 512 (tanh) -> 512 (relu) -> 10 (softmax + NLL)
# ---------------------------------------------------------------------------

def run_mlp(shim, dt, dims, acts, batch, seed, iters=1):
    from gpu_util import round_to
    rng = np.random.default_rng(seed)
    x = round_to(rng.uniform(0, 1, (dims[0], batch)), dt)
    labels = rng.integers(0, dims[-1], batch).astype(np.int32)
    Ws = [round_to(xavier(rng, dims[i + 1], dims[i]), dt) for i in range(len(acts))]
    bs = [round_to(xavier(rng, dims[i + 1], 1).reshape(-1), dt) for i in range(len(acts))]
    loss = np.zeros(1, np.float32)
    nll = np.zeros(batch, np.float32)
    dWs = [np.zeros(w.shape, np.float32, order="F") for w in Ws]
    dbs = [np.zeros(b.shape, np.float32) for b in bs]
    ms = ctypes.c_float(0)
    n = len(acts)
    check(shim, shim.scenario_mlp(
        dt, batch, n, (ctypes.c_int * (n + 1))(*dims), (ctypes.c_int * n)(*acts), fptr(f32(x)),
        labels.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), ptrs([f32(w) for w in Ws]), ptrs([f32(b) for b in bs]),
        iters, fptr(loss), fptr(nll), ptrs(dWs), ptrs(dbs), ctypes.byref(ms)))
    want = N.mlp_forward_backward(acts, [w.astype(np.float64) for w in Ws], [b.astype(np.float64) for b in bs],
                                  x.astype(np.float64), labels)
    return (loss[0], nll, dWs, dbs), want, ms.value


def test_mlp_fp32_full_config(shim):
    got, want, ms = run_mlp(shim, capi.F32, [784, 512, 512, 10], [N.TANH, N.RELU, N.IDENTITY], 64, seed=1, iters=3)
    loss, nll, dWs, dbs = got
    wloss, wnll, wdWs, wdbs = want
    assert abs(loss - wloss) <= 1e-4 * abs(wloss)
    assert rel_fro(nll, wnll) <= 1e-4
    for l in range(3):
        assert rel_fro(dWs[l], wdWs[l]) <= 1e-4, l
        assert rel_fro(dbs[l], wdbs[l]) <= 1e-4, l
    assert ms > 0


@pytest.mark.parametrize("dt", [capi.F16, capi.BF16])
@pytest.mark.parametrize("batch", [64, 7])
def test_mlp_16bit(shim, dt, batch):
    got, want, _ = run_mlp(shim, dt, [784, 512, 512, 10], [N.TANH, N.RELU, N.IDENTITY], batch, seed=2)
    loss, nll, dWs, dbs = got
    wloss, wnll, wdWs, wdbs = want
    assert abs(loss - wloss) <= 2e-2 * abs(wloss)
    assert rel_fro(nll, wnll) <= 2e-2
    for l in range(3):
        # every layer rounds its activations and gradients to 16 bits once more
        assert rel_fro(dWs[l], wdWs[l]) <= 4e-2, l
        assert rel_fro(dbs[l], wdbs[l]) <= 4e-2, l


@pytest.mark.parametrize("dims,acts,batch", [
    ([5, 4, 3], [N.SIGMOID, N.IDENTITY], 1),
    ([33, 65, 17, 9], [N.GELU, N.TANH, N.IDENTITY], 13),
    ([256, 256, 256], [N.RELU, N.IDENTITY], 256),
])
def test_mlp_fp32_shapes(shim, dims, acts, batch):
    got, want, _ = run_mlp(shim, capi.F32, dims, acts, batch, seed=len(dims))
    assert abs(got[0] - want[0]) <= 1e-4 * abs(want[0])
    for l in range(len(acts)):
        assert rel_fro(got[2][l], want[2][l]) <= 1e-4
        assert rel_fro(got[3][l], want[3][l]) <= 1e-4


# ---------------------------------------------------------------------------
# Autobatch: the reference's equivalence cases
# ---------------------------------------------------------------------------

def oracle_autobatch_case(which, vals):
    v = [a.astype(np.float64) for a in vals]
    if which == 0:
        x, y, b = v
        h, hpre = N.affine_forward(N.IDENTITY, [x, y, x, y, b])
        t, tpre = N.affine_forward(N.IDENTITY, [h, y, b])
        dt = np.ones_like(t)
        gt = N.affine_backward(N.IDENTITY, [h, y, b], t, tpre, dt)
        gh = N.affine_backward(N.IDENTITY, [x, y, x, y, b], h, hpre, gt[0])
        return t.sum(), [gh[0] + gh[2], gt[1] + gh[1] + gh[3], gt[2] + gh[4]]
    xs, (W, V, b) = v[:12], v[12:]
    act = N.TANH if which == 3 else N.IDENTITY
    grads = [np.zeros_like(a) for a in v]
    total = 0.0
    for i in range(3):
        h = np.zeros((3, 1))
        tape = []
        for t in range(4):
            ins = [W, xs[4 * i + t], V, h, b]
            h, pre = N.affine_forward(act, ins)
            tape.append((ins, h, pre))
        total += h.sum()
        dy = np.ones((3, 1))
        for t in range(3, -1, -1):
            ins, val, pre = tape[t]
            g = N.affine_backward(act, ins, val, pre, dy)
            grads[12] += g[0]
            grads[4 * i + t] += g[1]
            grads[13] += g[2]
            grads[14] += g[4].reshape(3, 1)
            dy = g[3]
    return total, grads


@pytest.fixture(params=[0, 1], ids=["cat", "gather"])
def gather(request, shim):
    """Autobatch as the reference rewrites (RowwiseCat + Prod + RowwiseUncat), and
    with one GatherProd per group (right operands and their gradients in place)."""
    shim.scenario_set_autobatch_gather(request.param)
    yield request.param
    shim.scenario_set_autobatch_gather(0)


@pytest.mark.parametrize("which", [0, 1, 2, 3])
def test_autobatch_reference_cases(shim, which, gather):
    rng = np.random.default_rng(40 + which)
    shapes = [(2, 2), (2, 2), (2,)] if which == 0 else [(2, 1)] * 12 + [(3, 2), (3, 3), (3, 1)]
    vals = [f32(rng.uniform(-1, 1, s)) for s in shapes]
    before, after = np.zeros(1, np.float32), np.zeros(1, np.float32)
    gb = [np.zeros(s, np.float32, order="F") for s in shapes]
    ga = [np.zeros(s, np.float32, order="F") for s in shapes]
    pb, pa = ctypes.c_int(0), ctypes.c_int(0)
    check(shim, shim.scenario_autobatch_case(which, ptrs(vals), fptr(before), fptr(after), ptrs(gb), ptrs(ga),
                                             ctypes.byref(pb), ctypes.byref(pa)))
    want, want_g = oracle_autobatch_case(which, vals)
    # Products by (left operand, height).  Case 0: x*y twice -> 1, h*y -> 1.  Recurrent cases: all twelve
    # W*x sit at one height -> 1; V*h has one height per step -> 4.  Case 3 is case 1 with tanh Affines: the
    # rewrite keeps the nonlinearity (the reference's drops it, ginn/autobatch.h:30-38).
    assert pa.value == (2 if which == 0 else 5)
    assert abs(before[0] - want) <= 1e-5 * max(1, abs(want))
    assert abs(after[0] - want) <= 1e-5 * max(1, abs(want))
    for i in range(len(shapes)):
        assert rel_fro(gb[i], want_g[i]) <= 1e-4, i
        assert rel_fro(ga[i], want_g[i]) <= 1e-4, i


# ---------------------------------------------------------------------------
# LSTM gates over ragged sequences, plain and autobatched
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("mode", [2, 6, 14, 22])
def test_mlp_level_executor(shim, mode):
    """The MLP through the level executor, also frozen after its first pass:
    same oracle, and the very results of node-by-node execution."""
    dims, acts = [784, 512, 512, 10], [N.TANH, N.RELU, N.IDENTITY]
    shim.scenario_set_executor(mode)
    try:
        got, want, _ = run_mlp(shim, capi.F32, dims, acts, 64, seed=7, iters=3)
    finally:
        shim.scenario_set_executor(0)
    plain, _, _ = run_mlp(shim, capi.F32, dims, acts, 64, seed=7, iters=3)
    assert abs(got[0] - want[0]) <= 1e-4 * abs(want[0])
    for l in range(3):
        assert rel_fro(got[2][l], want[2][l]) <= 1e-4, l
        assert rel_fro(got[3][l], want[3][l]) <= 1e-4, l
        np.testing.assert_array_equal(got[2][l], plain[2][l])
        np.testing.assert_array_equal(got[3][l], plain[3][l])
    assert got[0] == plain[0]


def run_lstm(shim, autobatch, lens, E, H, seed, iters=1):
    """autobatch is the scenario's mode: bit 0 = Autobatch rewrite, bit 1 = level executor,
    bit 2 = the executor is frozen after its first pass (the later ones replay the recorded plans),
    bit 3 = the frozen pass is recorded as a device graph and replayed."""
    rng = np.random.default_rng(seed)
    nseq, total = len(lens), int(sum(lens))
    W = f32(xavier(rng, 4 * H, E + H))
    b = f32(xavier(rng, 4 * H, 1).reshape(-1))
    xs = f32(rng.standard_normal((E, total)))
    mask = f32(rng.uniform(-1, 1, (H, nseq)))
    out_h = np.zeros((H, nseq), np.float32, order="F")
    loss = np.zeros(1, np.float32)
    dW, db, dxs = np.zeros_like(W), np.zeros_like(b), np.zeros_like(xs)
    ms, nodes, prods, launches = ctypes.c_float(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    check(shim, shim.scenario_lstm(
        autobatch, nseq, (ctypes.c_int * nseq)(*lens), E, H, fptr(W), fptr(b), fptr(xs), fptr(mask), iters,
        fptr(out_h), fptr(loss), fptr(dW), fptr(db), fptr(dxs), ctypes.byref(ms), ctypes.byref(nodes),
        ctypes.byref(prods), ctypes.byref(launches), None))
    offs = np.concatenate([[0], np.cumsum(lens)])
    xl = [np.asfortranarray(xs[:, offs[s]:offs[s + 1]].astype(np.float64)) for s in range(nseq)]
    W64, b64, m64 = W.astype(np.float64), b.astype(np.float64), mask.astype(np.float64)
    wh, _ = N.lstm_forward(W64, b64, xl)
    wdW, wdb, wdxs = N.lstm_backward(W64, b64, xl, m64)
    want = dict(h=wh, loss=float((wh * m64).sum()), dW=wdW, db=wdb, dxs=np.concatenate(wdxs, axis=1))
    got = dict(h=out_h, loss=float(loss[0]), dW=dW, db=db, dxs=dxs)
    return got, want, dict(ms=ms.value, nodes=nodes.value, prods=prods.value, launches=launches.value)


def compare_lstm(got, want):
    assert rel_fro(got["h"], want["h"]) <= 1e-4
    assert abs(got["loss"] - want["loss"]) <= 1e-4 * max(1.0, abs(want["loss"]))
    for key in ("dW", "db", "dxs"):
        assert rel_fro(got[key], want[key]) <= 1e-4, key


@pytest.mark.parametrize("autobatch", [0, 1])
@pytest.mark.parametrize("lens,E,H", [([3, 1, 4], 3, 2), ([5, 5, 5, 5], 8, 16), ([1], 4, 4),
                                       ([7, 2, 9, 4, 4, 1, 12, 6], 128, 256)])
def test_lstm_small(shim, autobatch, lens, E, H, gather):
    got, want, stats = run_lstm(shim, autobatch, lens, E, H, seed=len(lens))
    compare_lstm(got, want)
    if autobatch:
        # one product per time step at which at least two sequences are alive
        # + one per sequence step that runs alone
        steps = max(lens)
        alone = sum(1 for t in range(steps) if sum(1 for n in lens if n > t) == 1)
        merged = steps - alone
        assert stats["prods"] == merged + alone
    else:
        assert stats["prods"] == 0  # fused Affine nodes only


def test_lstm_autobatched_full_config(shim, gather):
    """256 sequences, lengths U{5..40}, embed 128, hidden 256."""
    rng = np.random.default_rng(2024)
    lens = rng.integers(5, 41, 256).tolist()
    got, want, stats = run_lstm(shim, 1, lens, 128, 256, seed=9)
    compare_lstm(got, want)
    assert stats["prods"] == max(lens)


@pytest.mark.parametrize("mode", [2, 3, 6, 7, 14, 15, 22, 23, 31])
@pytest.mark.parametrize("lens,E,H", [([3, 1, 4], 3, 2), ([5, 5, 5, 5], 8, 16), ([1], 4, 4),
                                       ([7, 2, 9, 4, 4, 1, 12, 6], 128, 256)])
def test_lstm_level_executor(shim, mode, lens, E, H, gather):
    """The same graphs through the level executor (element-wise nodes of one
    height share launches), plain (2) and after Autobatch (3): same oracle,
    same tolerance; against node-by-node execution only the order in which
    the users of a node add into its gradient differs (a few ulp).  Frozen
    (6, 7), the passes after the first replay the recorded launches: the very
    same results as asking every node again; 14, 15 replay them as one
    recorded device graph; 22, 23 join the table launches of consecutive levels
    into chain launches (one workgroup per independent chain of operations),
    31 replays that as a device graph: again the very same results -- but for the bias
    gradient, which a frozen pass sums in one reduction over the users of all levels at
    its end instead of one reduction per level (another order of the same additions)."""
    got, want, stats = run_lstm(shim, mode, lens, E, H, seed=len(lens), iters=2)
    compare_lstm(got, want)
    if mode & 4:
        thawed, _, _ = run_lstm(shim, mode & 3, lens, E, H, seed=len(lens), iters=2)
        for key in ("h", "dxs", "dW"):
            np.testing.assert_array_equal(got[key], thawed[key], err_msg=key)
        assert rel_fro(got["db"], thawed["db"]) <= 1e-6
    plain, _, _ = run_lstm(shim, mode & 1, lens, E, H, seed=len(lens))
    np.testing.assert_array_equal(got["h"], plain["h"])  # forward: the same arithmetic per element
    for key in ("dxs", "db", "dW"):
        assert rel_fro(got[key], plain[key]) <= 1e-6, key
    assert stats["launches"] > 0


def test_lstm_level_executor_full_config(shim, gather):
    """256 sequences, lengths U{5..40}: ~100 k nodes in a few thousand launches."""
    rng = np.random.default_rng(2024)
    lens = rng.integers(5, 41, 256).tolist()
    late = shim.scenario_late_sum_columns()
    got, want, stats = run_lstm(shim, 3, lens, 128, 256, seed=9)
    compare_lstm(got, want)
    assert stats["launches"] < stats["nodes"] / 10
    # With gathered products the weight gradient is ONE product per pass over the columns of all
    # steps (the warm-up pass and the timed one); with the reference's concatenation it is one per step.
    assert shim.scenario_late_sum_columns() - late == (2 * sum(lens) if gather else 0)
    got, want, stats = run_lstm(shim, 7, lens, 128, 256, seed=9, iters=3)
    compare_lstm(got, want)
    assert shim.scenario_timed_fills() == 0  # no gradient was zeroed on demand, one launch each
    fused, want, fstats = run_lstm(shim, 23, lens, 128, 256, seed=9, iters=3)
    compare_lstm(fused, want)
    assert shim.scenario_timed_fills() == 0
    for key in ("h", "dxs", "db", "dW"):
        np.testing.assert_array_equal(fused[key], got[key], err_msg=key)
    assert fstats["launches"] < stats["launches"] / 2
