"""The host layer's nodes on cpu(): Prod, BatchedProd, Affine (every epilogue) and the nonlinearity nodes run
the same graph code as on the device through the host layer's own loops (ginn_amd/ginn/cpu_ops.h), as the
reference's nodes do on its CPU device (ginn/node/prod.h:31-46, ginn/node/affine.h:49-53, ginn/nonlin.h).
Same cases, protocol (e = f() + f(), loss = Sum(mask * e)) and tolerances as tests/test_host_nodes_gpu.py,
against the numpy oracle; no GPU is touched."""
import ctypes

import numpy as np
import pytest

import test_host_nodes_gpu as G
from ginn_amd import capi
from oracle import nodes as N


@pytest.fixture(scope="module")
def cpu_shim():
    if not G.SHIM.exists():
        pytest.fail(f"{G.SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(G.SHIM))
    lib.shim_last_error.restype = ctypes.c_char_p
    lib.shim_use_device(1)
    yield lib
    lib.shim_use_device(0)


@pytest.mark.parametrize("dt", G.DTYPES)
@pytest.mark.parametrize("a_shape,b_shape,batched", [
    ((2, 3), (3, 2), 0), ((64, 48), (48, 33), 0), ((130, 70), (70, 96), 0), ((4, 6, 5), (30, 7), 0),
    # the packed product's edges: rows and columns that fill no register tile, sums across two K blocks
    ((37, 53), (53, 29), 0), ((300, 260), (260, 23), 0), ((17, 600), (600, 135), 0),
    ((2, 3, 4), (3, 5, 4), 1), ((2, 3, 2, 2), (3, 5, 2, 2), 1), ((64, 32, 8), (32, 48, 8), 1)])
def test_prod_nodes_on_cpu(cpu_shim, dt, a_shape, b_shape, batched):
    G.test_prod_nodes(cpu_shim, dt, a_shape, b_shape, batched)


@pytest.mark.parametrize("dt", G.DTYPES)
@pytest.mark.parametrize("act", [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.SOFTMAX, N.GELU, N.GELU2])
@pytest.mark.parametrize("case", ["vector", "broadcast", "high_rank", "two_pairs", "mlp_layer", "fixed_input"])
def test_affine_node_on_cpu(cpu_shim, dt, act, case):
    G.test_affine_node(cpu_shim, dt, act, case)


@pytest.mark.parametrize("dt", G.DTYPES)
@pytest.mark.parametrize("act", [N.IDENTITY, N.TANH, N.RELU, N.SIGMOID, N.SOFTMAX, N.GELU, N.GELU2, N.LOG, N.SQRT])
def test_nonlin_nodes_on_cpu(cpu_shim, dt, act):
    G.test_nonlin_nodes(cpu_shim, dt, act)


def test_reference_prod_golden_on_cpu(cpu_shim, golden):
    """W * V of test/nodes.cu.cpp:1023-1041 through ProdNode on cpu()."""
    G.test_prod_reference_golden(cpu_shim, golden, capi.F32)


def test_mlp_configuration_on_cpu():
    """The MLP configuration (batch 64, 784-512-512-10) forward + backward with its graph on cpu(), through
    the example graph that bench.py also times on the device: loss, per-example losses and all gradients
    against the oracle."""
    import bench
    from conftest import rel_fro
    dims, acts, batch, x, labels, Ws, bs = bench._mlp_case()
    ms, loss, nll, dWs, dbs = bench.mlp_on_host_nodes(1)
    want_loss, want_nll, want_dW, want_db = N.mlp_forward_backward(acts, Ws, bs, x, labels)
    assert ms > 0
    assert abs(float(loss[0]) - want_loss) <= 1e-4 * abs(want_loss)
    assert rel_fro(nll, want_nll) <= 1e-4
    for got, ref in zip(dWs + dbs, list(want_dW) + list(want_db)):
        assert rel_fro(got, np.asarray(ref).reshape(got.shape)) <= 1e-4


@pytest.fixture(scope="module")
def cpu_scenarios():
    """libginn_examples.so with its graphs placed on cpu() (scenario_set_device)."""
    import test_scenarios_gpu as S
    if not S.SHIM.exists():
        pytest.fail(f"{S.SHIM} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(S.SHIM))
    lib.scenario_last_error.restype = ctypes.c_char_p
    lib.scenario_timed_fills.restype = ctypes.c_long
    lib.scenario_set_executor(0)
    lib.scenario_set_device(1)
    yield lib
    lib.scenario_set_device(0)


@pytest.mark.parametrize("lens,E,H", [([3, 1, 4], 3, 2), ([5, 5, 5, 5], 8, 16), ([1], 4, 4),
                                       ([7, 2, 9, 4, 4, 1, 12, 6], 128, 256)])
def test_lstm_graph_on_cpu(cpu_scenarios, lens, E, H):
    """The LSTM configuration's graph (Slice, Cat, Affine, gates, CwiseProd, Add, RowwiseCat, Sum) node by node
    on cpu(): final states, loss and the gradients of W, b and the inputs against the oracle."""
    import test_scenarios_gpu as S
    got, want, stats = S.run_lstm(cpu_scenarios, 0, lens, E, H, seed=len(lens))
    S.compare_lstm(got, want)
    assert stats["prods"] == 0


@pytest.mark.parametrize("C,nh,B,T,V", [(12, 3, 2, 5, 11), (64, 4, 3, 33, 50)])
def test_gpt_layer_graph_on_cpu(cpu_scenarios, C, nh, B, T, V):
    """The GPT layer's graph (LayerNorm + gamma / beta, projections, Reshape / Permute, BatchedProd, the in-place
    scale and mask, Softmax, residuals, GELU MLP, head, PickNegLogSoftmax, Mean) node by node on cpu(): loss and
    all 21 gradients against the oracle."""
    import test_seqops_gpu as Q
    loss, got, wloss, want, _ = Q.run_gpt(cpu_scenarios, capi.F32, C, nh, B, T, V, seed=C, wscale=0.2)
    assert abs(loss - wloss) <= 1e-4 * abs(wloss)
    errs = Q.grad_errors(got, want)
    assert max(errs.values()) <= 1e-4, errs
