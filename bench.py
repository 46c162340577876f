#!/usr/bin/env python3
"""Headline benchmark: fp16 (fp32-accumulate) column-major GEMM, M = N = K = 8192,
through the C ABI (`ginn_hip_gemm`), one GPU.

A "step" is one product C = A * B (NN) on operands already resident in HBM.
Prints ONE JSON line on stdout:

  value        whole-job TFLOP/s = 2 M N K * steps / wall time of the timed region
  roofline     the product kernel against the MI355X dense fp16 MFMA peak,
               timed with HIP events on the stream the kernel runs on
  cpu_baseline the CPU oracle's blocked fp32 product, one thread, on a bounded
               column panel of the same product (a reported baseline only)

Other workloads of the build target (`--workload`) reuse the same harness;
`--report FILE` additionally writes the whole sweep as JSON.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time
from ctypes import byref, c_float, c_void_p
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_TFLOPS = {"f16": 2500.0, "bf16": 2500.0, "f32": 157.3}
PEAK_HBM_GBS = 8000.0
# HBM bytes per launch (FETCH_SIZE + WRITE_SIZE, scaled by a copy kernel of known size) come from
# rocprofv3 --pmc runs, not from this process: profiles/hbm_traffic.txt lists them, one workload per line,
# with the summary file that documents the run.
TRAFFIC_FILE = ROOT / "profiles" / "hbm_traffic.txt"
# Untimed launches in front of --warmup: the clocks of an idle part take ~0.1 s of this kernel to ramp.
RAMP_SECONDS = 0.3
DT = {"f32": 0, "f16": 1, "bf16": 2}
ESIZE = {"f32": 4, "f16": 2, "bf16": 2}


def parse_args():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    # The first ~70 launches of a session run while the clocks ramp up (946 -> 1220 TFLOP/s over the
    # first 0.1 s on the headline shape): the default warm-up is long enough to time the steady state.
    p.add_argument("--steps", type=int, default=100)
    p.add_argument("--warmup", type=int, default=100)
    p.add_argument("--workload", default="gemm",
                   help="gemm (headline) | sweep (all GEMM shapes of the build target) | "
                        "configs (MLP, autobatched LSTM, attention products, GPT layer: GPU time with the CPU "
                        "oracle beside) | mlp | lstm | attention | gpt | update (one of those alone, for profiling) | "
                        "ragged (products whose extents are no multiples of the tiles) | "
                        "skinny (narrow right-hand sides against the HBM roofline) | "
                        "copy (a plain copy kernel of known size, to calibrate the HBM counters)")
    p.add_argument("--dtype", default="f16", choices=list(DT))
    p.add_argument("--layout", default="NN", choices=["NN", "NT", "TN"])
    p.add_argument("--size", type=int, default=8192)
    p.add_argument("--n", type=int, default=0, help="N if different from --size (skinny shapes)")
    p.add_argument("--beta", type=float, default=0.0)
    p.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    p.add_argument("--no-ramp", action="store_true", help="skip the untimed clock ramp in front of --warmup")
    p.add_argument("--no-configs", action="store_true",
                   help="skip the MLP / LSTM / GPT-layer passes that fill the `configs` block")
    p.add_argument("--cpu-panel", type=int, default=8192,
                   help="columns of the product that the CPU baseline computes")
    p.add_argument("--report", default="", help="write the sweep results to this JSON file")
    return p.parse_args()


class Harness:
    def __init__(self):
        import torch
        from ginn_amd import capi
        if not torch.cuda.is_available():
            raise SystemExit("bench.py needs a GPU (no CPU fallback exists)")
        self.torch, self.capi = torch, capi
        self.lib = capi.load()
        self.ctx = self.lib.ctx_create(0)
        torch.cuda.set_device(0)

    def tdtype(self, name):
        t = self.torch
        return {"f32": t.float32, "f16": t.float16, "bf16": t.bfloat16}[name]

    def operands(self, dtype, layout, m, n, k, seed=0):
        """Column-major operands as stored: NN A[m x k], B[k x n]; NT B stored
        [n x k]; TN A stored [k x m].  Entries N(0,1)/sqrt(k)."""
        t = self.torch
        g = t.Generator(device="cuda").manual_seed(seed)
        s = 1.0 / (k ** 0.5)
        a_rows, a_cols = (k, m) if layout[0] == "T" else (m, k)
        b_rows, b_cols = (n, k) if layout[1] == "T" else (k, n)
        A = (t.randn(a_cols, a_rows, generator=g, device="cuda") * s).to(self.tdtype(dtype))
        B = (t.randn(b_cols, b_rows, generator=g, device="cuda") * s).to(self.tdtype(dtype))
        C = t.zeros(n, m, device="cuda", dtype=self.tdtype(dtype))
        t.cuda.synchronize()
        return A, B, C, a_rows, b_rows

    def time_gemm(self, dtype, layout, m, n, k, steps, warmup, beta=0.0, ramp_seconds=0.0):
        A, B, C, lda, ldb = self.operands(dtype, layout, m, n, k)
        op_a, op_b = int(layout[0] == "T"), int(layout[1] == "T")
        lib, ctx = self.lib, self.ctx
        args = (ctx, DT[dtype], op_a, op_b, m, n, k, c_void_p(A.data_ptr()), lda,
                c_void_p(B.data_ptr()), ldb, beta, c_void_p(C.data_ptr()), m)
        # Time-bounded, untimed ramp: the same launches until ramp_seconds have passed, whatever --warmup is.
        self.ramp_launches = 0
        t_end = time.perf_counter() + ramp_seconds
        while ramp_seconds > 0 and time.perf_counter() < t_end:
            for _ in range(8):
                lib.call("ginn_hip_gemm", *args)
            lib.call("ginn_hip_sync", ctx)
            self.ramp_launches += 8
        for _ in range(warmup):
            lib.call("ginn_hip_gemm", *args)
        lib.call("ginn_hip_sync", ctx)
        self.torch.cuda.synchronize()
        t0 = time.perf_counter()
        lib.call("ginn_hip_event_record", ctx, 0)
        for _ in range(steps):
            lib.call("ginn_hip_gemm", *args)
        lib.call("ginn_hip_event_record", ctx, 1)
        lib.call("ginn_hip_sync", ctx)
        self.torch.cuda.synchronize()
        wall = time.perf_counter() - t0
        ms = c_float(0)
        lib.call("ginn_hip_event_elapsed_ms", ctx, 0, 1, byref(ms))
        return wall, ms.value / steps, C


# ---------------------------------------------------------------------------
# The other configurations of the build target (graph level, through the C++
# host layer compiled into libginn_examples.so; attention through the C ABI)
# ---------------------------------------------------------------------------

FP = ctypes.POINTER(ctypes.c_float)


def _f32(a):
    import numpy as np
    return np.asfortranarray(a, dtype=np.float32)


def _fp(a):
    return a.ctypes.data_as(FP)


def _examples():
    from ginn_amd import capi
    path = capi.LIB_PATH.parent / "libginn_examples.so"
    if not path.exists():
        raise SystemExit(f"{path} is missing: run __graft_entry__.build()")
    capi.load()
    lib = ctypes.CDLL(str(path))
    lib.scenario_last_error.restype = ctypes.c_char_p
    return lib


def _cpu_timed(fn):
    """Runs fn on one thread (the reference's Eigen build is single threaded)."""
    from threadpoolctl import threadpool_limits
    with threadpool_limits(limits=1):
        t0 = time.perf_counter()
        fn()
        return (time.perf_counter() - t0) * 1e3


def _xavier(rng, rows, cols):
    import numpy as np
    a = np.sqrt(6.0 / (0.5 * (rows + cols)))
    return rng.uniform(-a, a, (rows, cols))


def _mlp_case():
    """Inputs of the MLP configuration: fp32, batch 64, 784 -> 512 tanh -> 512 relu -> 10."""
    import numpy as np
    from ginn_amd import capi
    rng = np.random.default_rng(1)
    dims, acts, batch = [784, 512, 512, 10], [capi.ACT_TANH, capi.ACT_RELU, capi.ACT_IDENTITY], 64
    x = _f32(rng.uniform(0, 1, (dims[0], batch)))
    labels = rng.integers(0, 10, batch).astype(np.int32)
    Ws = [_f32(_xavier(rng, dims[i + 1], dims[i])) for i in range(3)]
    bs = [_f32(_xavier(rng, dims[i + 1], 1).reshape(-1)) for i in range(3)]
    return dims, acts, batch, x, labels, Ws, bs


def _run_mlp(ex, iters, case):
    """scenario_mlp on `case`: (ms per pass, loss, per-example losses, dW, db)."""
    import numpy as np
    dims, acts, batch, x, labels, Ws, bs = case
    dWs, dbs = [np.zeros_like(w) for w in Ws], [np.zeros_like(b) for b in bs]
    loss, nll, ms = np.zeros(1, np.float32), np.zeros(batch, np.float32), ctypes.c_float(0)
    rc = ex.scenario_mlp(0, batch, 3, (ctypes.c_int * 4)(*dims), (ctypes.c_int * 3)(*acts), _fp(x),
                         labels.ctypes.data_as(ctypes.POINTER(ctypes.c_int)), (FP * 3)(*map(_fp, Ws)),
                         (FP * 3)(*map(_fp, bs)), iters, _fp(loss), _fp(nll), (FP * 3)(*map(_fp, dWs)),
                         (FP * 3)(*map(_fp, dbs)), ctypes.byref(ms))
    if rc:
        raise SystemExit(ex.scenario_last_error().decode())
    return ms.value, loss, nll, dWs, dbs


def mlp_on_host_nodes(iters):
    """The MLP configuration forward + backward with its graph on cpu(): the same example graph as on the
    device, run node by node through the host layer's own loops (ginn_amd/ginn/cpu_ops.h, one thread).
    Returns (ms per pass, loss, per-example losses, dW, db); touches no GPU."""
    ex = _examples()
    ex.scenario_set_executor(0)
    ex.scenario_set_device(1)
    try:
        return _run_mlp(ex, iters, _mlp_case())
    finally:
        ex.scenario_set_device(0)


def bench_mlp(iters, cpu, executor=6):
    """MLP of AffineNodes, fp32, batch 64, 784 -> 512 tanh -> 512 relu -> 10, Sum(PickNegLogSoftmax).
    executor: 0 = Graph (node by node), 2 = level executor, 6 = level executor frozen after its first pass,
    14 = the frozen pass recorded as a device graph."""
    ex = _examples()
    ex.scenario_set_executor(executor)
    case = _mlp_case()
    dims, acts, batch, x, labels, Ws, bs = case
    ms = _run_mlp(ex, iters, case)[0]
    flops = 3 * sum(2.0 * dims[i + 1] * dims[i] * batch for i in range(3)) - 2.0 * 512 * 784 * batch
    ex.scenario_set_executor(0)
    # Algorithmic bytes of the pass: 4 (M K + K N + M N (1 + beta)) over its eight products (three forward,
    # three dW = dpre X^T, two dX = W^T dpre: the input takes no gradient), beta = 0 throughout.
    by = 0.0
    for i in range(3):
        mm, kk = dims[i + 1], dims[i]
        per = 4.0 * (mm * kk + kk * batch + mm * batch)
        by += per * (3 if i else 2)
    r = {"config": f"mlp fp32 b64 784-512-512-10 fwd+bwd, executor={executor}", "gpu_ms": round(ms, 4),
         "gflops": round(flops / ms / 1e6, 1), "gbs": round(by / ms / 1e6, 1), "algorithmic_bytes": int(by)}
    if executor & 8:
        r["kernels_per_pass"] = int(ex.scenario_recorded_kernels())
    if cpu:
        from oracle import nodes as N
        r["cpu_ms"] = round(_cpu_timed(lambda: N.mlp_forward_backward(acts, Ws, bs, x, labels)), 3)
        r["cpu"] = "oracle (numpy fp32 restatement), 1 thread"
        r["cpu_nodes_ms"] = round(mlp_on_host_nodes(10)[0], 3)
        r["cpu_nodes"] = "the same graph on cpu(): host layer nodes over their own fp32 loops, 1 thread"
    return r


def bench_lstm(iters, cpu, mode=7, gather=False):
    """LSTM gates, fp32: 256 sequences, lengths U{5..40}, embed 128, hidden 256.
    mode: bit 0 = Autobatch rewrite (products merged), bit 1 = level executor
    (element-wise nodes of one height share launches), bit 2 = executor frozen
    after its first pass (the timed passes replay the recorded launches; without
    it every node is asked again in every pass), bit 3 = the frozen pass recorded
    as a device graph (one graph launch per pass), bit 4 = the table launches of
    consecutive levels joined into chain launches.  gather: Autobatch merges a
    group into one GatherProd (right operands read, and their gradients added,
    where they are) instead of RowwiseCat + Prod + RowwiseUncat."""
    import numpy as np
    ex = _examples()
    ex.scenario_set_autobatch_gather(1 if gather else 0)
    rng = np.random.default_rng(2024)
    nseq, E, H = 256, 128, 256
    lens = rng.integers(5, 41, nseq).tolist()
    total = int(sum(lens))
    W = _f32(_xavier(rng, 4 * H, E + H))
    b = _f32(_xavier(rng, 4 * H, 1).reshape(-1))
    xs = _f32(rng.standard_normal((E, total)))
    mask = _f32(rng.uniform(-1, 1, (H, nseq)))
    out_h, loss = np.zeros((H, nseq), np.float32, order="F"), np.zeros(1, np.float32)
    dW, db, dxs = np.zeros_like(W), np.zeros_like(b), np.zeros_like(xs)
    ms, nodes, prods, launches = ctypes.c_float(0), ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    first_ms = ctypes.c_float(0)
    rc = ex.scenario_lstm(mode, nseq, (ctypes.c_int * nseq)(*lens), E, H, _fp(W), _fp(b), _fp(xs), _fp(mask),
                          iters, _fp(out_h), _fp(loss), _fp(dW), _fp(db), _fp(dxs), ctypes.byref(ms),
                          ctypes.byref(nodes), ctypes.byref(prods), ctypes.byref(launches), ctypes.byref(first_ms))
    ex.scenario_set_autobatch_gather(0)
    if rc:
        raise SystemExit(ex.scenario_last_error().decode())
    flops = 3 * 2.0 * 4 * H * (E + H) * total
    # Algorithmic bytes of the pass: per time step t with n_t sequences alive, the merged products
    # Z = W X_t and dX_t = W^T dZ_t (4 (M K + K n_t + M n_t) each), and once the weight gradient over all
    # columns (4 (M total + K total + M K)).
    M_, K_ = 4 * H, E + H
    alive = [sum(1 for L in lens if L > t) for t in range(max(lens))]
    by = sum(2 * 4.0 * (M_ * K_ + K_ * n_t + M_ * n_t) for n_t in alive) + 4.0 * (M_ * total + K_ * total + M_ * K_)
    r = {"config": f"lstm gates fp32 256 seqs (sum len {total}) E128 H256 fwd+bwd, autobatch={('gather' if gather else 'cat') if mode & 1 else 0}, "
                   f"level executor={(mode >> 1) & 1}, frozen={(mode >> 2) & 1}, device graph={(mode >> 3) & 1}, "
                   f"chains={(mode >> 4) & 1}",
         "gpu_ms": round(ms.value, 3), "gflops": round(flops / ms.value / 1e6, 1), "graph_nodes": nodes.value,
         "products": prods.value, "table_launches_per_pass": launches.value,
         "first_pass_ms": round(first_ms.value, 2), "gbs": round(by / ms.value / 1e6, 1),
         "algorithmic_bytes": int(by)}
    if mode & 8:
        r["kernels_per_pass"] = int(ex.scenario_recorded_kernels())
    if cpu:
        from oracle import nodes as N
        offs = np.concatenate([[0], np.cumsum(lens)])
        xl = [np.asfortranarray(xs[:, offs[s]:offs[s + 1]]) for s in range(nseq)]
        r["cpu_ms"] = round(_cpu_timed(lambda: N.lstm_backward(W, b, xl, mask)), 2)
        r["cpu"] = "oracle (numpy fp32, sequences batched per step), 1 thread"
        # The same graph with its nodes on cpu(): node by node through the host layer's own loops (no Autobatch,
        # one Affine per sequence step, as the reference runs it on its CPU device), one pass.
        ex.scenario_set_device(1)
        try:
            cms = ctypes.c_float(0)
            rc = ex.scenario_lstm(0, nseq, (ctypes.c_int * nseq)(*lens), E, H, _fp(W), _fp(b), _fp(xs), _fp(mask),
                                  1, _fp(out_h), _fp(loss), _fp(dW), _fp(db), _fp(dxs), ctypes.byref(cms),
                                  ctypes.byref(nodes), ctypes.byref(prods), ctypes.byref(launches), None)
        finally:
            ex.scenario_set_device(0)
        if rc:
            raise SystemExit(ex.scenario_last_error().decode())
        r["cpu_nodes_ms"] = round(cms.value, 1)
        r["cpu_nodes"] = "the same graph on cpu(): host layer nodes, one Affine per sequence step, 1 thread"
    return r


def bench_attention(h, steps, warmup, cpu, store_floor=False):
    """BatchedProd attention products, fp16: batch 128, QK^T [256x64][64x256] and PV [256x256][256x64],
    forward and both backward products of each.  store_floor: one more line, a plain fill of the 16.8 MB
    that the two products with a [256 x 256] result store -- what writing those bytes costs with no operand
    read and no arithmetic, launch included."""
    import numpy as np
    t = h.torch
    cases = [("QK^T fwd  NN", 0, 0, 256, 256, 64), ("QK^T dK   NT", 0, 1, 256, 64, 256),
             ("QK^T dQ   TN", 1, 0, 64, 256, 256), ("PV   fwd  NN", 0, 0, 256, 64, 256),
             ("PV   dP   NT", 0, 1, 256, 256, 64), ("PV   dV   TN", 1, 0, 256, 64, 256)]
    out = []
    batch = 128
    ex = _examples()
    for name, op_a, op_b, m, n, k in cases:
        ar, ac = (k, m) if op_a else (m, k)
        br, bc = (n, k) if op_b else (k, n)
        A = (t.randn(batch, ac, ar, device="cuda") / k ** 0.5).half()
        B = (t.randn(batch, bc, br, device="cuda") / k ** 0.5).half()
        C = t.zeros(batch, n, m, device="cuda", dtype=t.float16)
        args = (h.ctx, DT["f16"], op_a, op_b, m, n, k, c_void_p(A.data_ptr()), ar, ctypes.c_longlong(ar * ac),
                c_void_p(B.data_ptr()), br, ctypes.c_longlong(br * bc), c_float(0.0), c_void_p(C.data_ptr()), m,
                ctypes.c_longlong(m * n), batch)
        t.cuda.synchronize()
        # Issued from native code (libginn_examples.so), so that the calls reach the stream faster than
        # they run; the first product of a run meets clocks that are still rising, so every product is
        # timed twice and the second time counts.
        ms = c_float(0)
        if not out:
            # Untimed ramp in front of the first product: memory and fabric clocks of an idle part (or
            # one that ran launch-bound work before) take some tenths of a second of this traffic to rise.
            t_end = time.perf_counter() + 0.3
            while time.perf_counter() < t_end:
                ex.scenario_time_batched_gemm(*args, 0, 200, byref(ms))
        for _ in range(2):
            rc = ex.scenario_time_batched_gemm(*args, warmup, steps, byref(ms))
            if rc != 0:
                raise SystemExit(f"scenario_time_batched_gemm: {ex.scenario_last_error().decode()}")
        ms = ms.value
        fl, by = 2.0 * m * n * k * batch, 2.0 * (m * k + k * n + m * n) * batch
        r = {"config": f"attention fp16 batch 128 {name} m{m} n{n} k{k}", "gpu_ms": round(ms, 5),
             "tflops": round(fl / ms / 1e9, 2), "gbs": round(by / ms / 1e6, 1),
             "frac_hbm": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
        if cpu:
            from oracle import cgemm
            rng = np.random.default_rng(0)
            a = np.asfortranarray(rng.standard_normal((ar, ac, batch), dtype=np.float32))
            b = np.asfortranarray(rng.standard_normal((br, bc, batch), dtype=np.float32))
            r["cpu_ms"] = round(_cpu_timed(lambda: cgemm.bgemm(a, b, op_a=op_a, op_b=op_b, kind="f32", threads=1)), 2)
            r["cpu"] = "oracle_bgemm_f32, 1 thread"
        out.append(r)
    if store_floor:
        n = batch * 256 * 256
        buf = t.empty(n, device="cuda", dtype=t.float16)
        ms = c_float(0)
        for _ in range(2):
            for i in range(warmup + steps):
                if i == warmup:
                    h.lib.call("ginn_hip_event_record", h.ctx, 0)
                h.lib.call("ginn_hip_fill", h.ctx, DT["f16"], c_void_p(buf.data_ptr()), n, c_float(1.0))
            h.lib.call("ginn_hip_event_record", h.ctx, 1)
            h.lib.call("ginn_hip_sync", h.ctx)
            h.lib.call("ginn_hip_event_elapsed_ms", h.ctx, 0, 1, byref(ms))
        ms = ms.value / steps
        out.append({"config": "fill of 16.8 MB fp16 (the bytes a [256 x 256] x 128 result stores; calls issued from "
                              "Python, see the kernel trace for the kernel alone)", "gpu_ms": round(ms, 5),
                    "gbs": round(2.0 * n / ms / 1e6, 1), "frac_hbm": round(2.0 * n / ms / 1e6 / PEAK_HBM_GBS, 4)})
    return out


def time_product(h, dtype, layout, m, n, k, steps, warmup, batch=1):
    """Milliseconds per product (HIP events on the context's stream around back-to-back launches issued from
    native code, so that launches of a few microseconds are not bound by the interpreter); goes through
    ginn_hip_gemm_strided_batched, which with one slice selects kernels exactly as ginn_hip_gemm does."""
    t = h.torch
    g = t.Generator(device="cuda").manual_seed(0)
    lda, a_cols = (k, m) if layout[0] == "T" else (m, k)
    ldb, b_cols = (n, k) if layout[1] == "T" else (k, n)
    A = (t.randn(batch, a_cols, lda, generator=g, device="cuda") / k ** 0.5).to(h.tdtype(dtype))
    B = (t.randn(batch, b_cols, ldb, generator=g, device="cuda") / k ** 0.5).to(h.tdtype(dtype))
    C = t.zeros(batch, n, m, device="cuda", dtype=h.tdtype(dtype))
    t.cuda.synchronize()
    ex = _examples()
    ms = c_float(0)
    args = (h.ctx, DT[dtype], int(layout[0] == "T"), int(layout[1] == "T"), m, n, k, c_void_p(A.data_ptr()), lda,
            ctypes.c_longlong(lda * a_cols), c_void_p(B.data_ptr()), ldb, ctypes.c_longlong(ldb * b_cols), c_float(0.0),
            c_void_p(C.data_ptr()), m, ctypes.c_longlong(m * n), batch)
    for _ in range(2):  # the second measurement counts: the first meets clocks that are still moving
        if ex.scenario_time_batched_gemm(*args, warmup, steps, byref(ms)) != 0:
            raise SystemExit(f"scenario_time_batched_gemm: {ex.scenario_last_error().decode()}")
    return ms.value


def bench_ragged(h, steps, warmup):
    """Products whose extents are no multiples of the kernels' tiles: the shapes of the reference's own
    benchmark (4000^3, 1000^3, 16000 x 16000 x 4000: examples/bench.cu.cpp:216-220), a vocabulary of 50 264
    rows beside one of 50 304, and the attention products of a sequence length of 504 beside 512."""
    cases = [("f16", "NN", 4000, 4000, 4000, 1), ("f16", "NT", 4000, 4000, 4000, 1), ("f16", "TN", 4000, 4000, 4000, 1),
             ("f16", "NN", 4096, 4096, 4096, 1), ("f16", "NN", 2000, 2000, 2000, 1), ("f16", "NN", 1000, 1000, 1000, 1),
             ("f16", "NN", 16000, 16000, 4000, 1), ("f32", "NN", 4000, 4000, 4000, 1), ("f32", "NN", 1000, 1000, 1000, 1),
             ("bf16", "NN", 50264, 4096, 768, 1), ("bf16", "NN", 50304, 4096, 768, 1),
             ("bf16", "NT", 50264, 768, 4096, 1), ("bf16", "NT", 50304, 768, 4096, 1),
             ("bf16", "NN", 504, 504, 64, 96), ("bf16", "NN", 512, 512, 64, 96),
             ("bf16", "NN", 64, 504, 504, 96), ("bf16", "NN", 64, 512, 512, 96),
             ("bf16", "NT", 504, 64, 504, 96), ("bf16", "TN", 64, 504, 504, 96)]
    time_product(h, "f16", "NN", 8192, 8192, 8192, 100, 100)  # untimed: lets the clocks settle
    out = []
    for dt, lay, m, n, k, batch in cases:
        fl = 2.0 * m * n * k * batch
        ms = time_product(h, dt, lay, m, n, k, max(5, min(steps, int(4e12 / fl) + 5)), warmup, batch)
        by = ESIZE[dt] * (m * k + k * n + m * n) * batch
        out.append({"config": f"{dt} {lay} {m}x{n}x{k}" + (f" x {batch} slices" if batch > 1 else ""),
                    "us": round(ms * 1e3, 2), "tflops": round(fl / ms / 1e9, 1),
                    "frac_mfma": round(fl / ms / 1e9 / PEAK_TFLOPS[dt], 4), "gbs": round(by / ms / 1e6, 1)})
    return out


def bench_skinny(h, steps, warmup):
    """NN products with a narrow right-hand side, against the HBM roofline (A is read once): the skinny
    shapes of the GEMM sweep (M = K = 4096, N = 1, 16, 64) and tall products over a smaller A, which run as
    one launch (16-row strips over all of K) instead of a split of K plus a fold."""
    cases = [(dt, 4096, n, 4096) for dt in ("f32", "f16", "bf16") for n in (1, 16, 64)]
    cases += [("f16", 4096, 1, 1024), ("f16", 4096, 16, 1024), ("f16", 4096, 16, 2048), ("f16", 2048, 4, 2048),
              ("f16", 2048, 1, 4096), ("f32", 4096, 16, 1024), ("f32", 4096, 16, 2048)]
    time_product(h, "f16", "NN", 8192, 8192, 8192, 100, 100)  # untimed: lets the clocks settle
    out = []
    for dt, m, n, k in cases:
        ms = time_product(h, dt, "NN", m, n, k, steps, warmup)
        by = ESIZE[dt] * (m * k + k * n + m * n)
        out.append({"config": f"{dt} NN {m}x{n}x{k}", "us": round(ms * 1e3, 2), "gbs": round(by / ms / 1e6, 1),
                    "frac_hbm": round(by / ms / 1e6 / PEAK_HBM_GBS, 4),
                    "frac_mfma": round(2.0 * m * n * k / ms / 1e9 / PEAK_TFLOPS[dt], 4)})
    return out


def bench_update(h, steps, warmup, cpu):
    """One Adam / SGD step (ginn/update/update.h:54-133) over the weights of the GPT configuration (one
    decoder layer + vocabulary head, d 768, MLP 3072, vocab 8192: 13.4 M parameters in 14 tensors) in one
    launch, and over one 64 Mi-element weight.  Memory-bound: Adam reads w, g, m, v and writes w, m, v."""
    import numpy as np
    from ginn_amd import capi
    t = h.torch
    C, F, V = 768, 3072, 8192
    gpt = [C * 3 * C, 3 * C, C * C, C, F * C, F, C * F, C, C, C, C, C, V * C, V]
    out = []
    for label, sizes, dtype in [("gpt layer + head, 14 weights", gpt, "f32"), ("gpt layer + head, 14 weights", gpt, "bf16"),
                                ("one weight of 64 Mi elements", [1 << 26], "f32")]:
        for kind, name in [(capi.UPDATE_ADAM, "adam"), (capi.UPDATE_SGD, "sgd")]:
            ws = [t.randn(n, device="cuda").to(h.tdtype(dtype)) for n in sizes]
            gs = [(t.randn(n, device="cuda") * 0.1).to(h.tdtype(dtype)) for n in sizes]
            ms_ = [t.zeros(n, device="cuda") for n in sizes]
            vs = [t.zeros(n, device="cuda") for n in sizes]
            adam = kind == capi.UPDATE_ADAM
            ops = (capi.UpdateOp * len(sizes))(*[
                capi.UpdateOp(w.data_ptr(), g.data_ptr(), m.data_ptr() if adam else None, v.data_ptr() if adam else None,
                              n, DT[dtype], 0) for w, g, m, v, n in zip(ws, gs, ms_, vs, sizes)])
            table = t.from_numpy(np.frombuffer(bytes(ops), dtype=np.uint8).copy()).cuda()
            rule = capi.UpdateRule(kind, 1e-3, 5.0, 0.9, 0.1, 0.999, 0.001, -1e-2, 1000.0, 1e-8)
            args = (h.ctx, byref(rule), len(sizes), c_void_p(table.data_ptr()), max(sizes))
            t.cuda.synchronize()
            for _ in range(warmup):
                h.lib.call("ginn_hip_multi_update", *args)
            h.lib.call("ginn_hip_event_record", h.ctx, 0)
            for _ in range(steps):
                h.lib.call("ginn_hip_multi_update", *args)
            h.lib.call("ginn_hip_event_record", h.ctx, 1)
            h.lib.call("ginn_hip_sync", h.ctx)
            ms = c_float(0)
            h.lib.call("ginn_hip_event_elapsed_ms", h.ctx, 0, 1, byref(ms))
            ms = ms.value / steps
            es = ESIZE[dtype]
            total = sum(sizes)
            # algorithmic bytes: w and g read, w written (+ m, v read and written for Adam); the clipped
            # gradient goes back only where clipping changed it (nowhere here)
            by = total * (3 * es + (16 if adam else 0))
            r = {"config": f"{name} step, {dtype} weights, {label} ({total} elements)", "gpu_ms": round(ms, 5),
                 "gbs": round(by / ms / 1e6, 1), "frac_hbm": round(by / ms / 1e6 / PEAK_HBM_GBS, 4),
                 "bytes_per_launch": by}
            if cpu and adam and dtype == "f32" and len(sizes) > 1:
                from oracle import update as U
                rng = np.random.default_rng(0)
                cw = [rng.standard_normal(n).astype(np.float32) for n in sizes]
                cg = [rng.standard_normal(n).astype(np.float32) * 0.1 for n in sizes]
                o = U.Adam()

                def step():
                    for i in range(len(sizes)):
                        cw[i], _ = o.update(cw[i], cg[i], i)
                r["cpu_ms"] = round(_cpu_timed(step), 2)
                r["cpu"] = "oracle (numpy fp32, one expression at a time as the reference's Eigen), 1 thread"
            out.append(r)
            del ws, gs, ms_, vs
    return out


def bench_gpt(iters, cpu, dtype="bf16", executor=6, train=None):
    """GPT decoder layer fwd+bwd: d_model 768, 12 heads, seq 512, batch 8, MLP 3072, vocab 8192.
    executor: 0 = Graph (node by node), 2 = level executor, 6 = level executor frozen after its first pass,
    14 = the frozen pass recorded as a device graph.  train: None, or "adam" / "sgd": every pass
    ends with the update of all 20 weights (one launch), i.e. a whole training step is timed."""
    import numpy as np
    from ginn_amd import capi
    ex = _examples()
    ex.scenario_set_executor(executor)
    ex.scenario_set_training({None: -1, "sgd": 0, "adam": 1}[train], ctypes.c_float(1e-4), ctypes.c_float(5.0))
    rng = np.random.default_rng(5)
    C, nh, B, T, V = 768, 12, 8, 512, 8192
    shapes = dict(ln1_g=(C,), ln1_b=(C,), Wk=(C, C), bk=(C,), Wq=(C, C), bq=(C,), Wv=(C, C), bv=(C,), Wp=(C, C),
                  bp=(C,), ln2_g=(C,), ln2_b=(C,), W1=(4 * C, C), b1=(4 * C,), W2=(C, 4 * C), b2=(C,), lnf_g=(C,),
                  lnf_b=(C,), Wh=(V, C), bh=(V,))
    params = {k: _f32(rng.standard_normal(s) * 0.02) for k, s in shapes.items()}
    x = _f32(rng.standard_normal((C, B, T)))
    targets = rng.integers(0, V, B * T).astype(np.int32)
    pin = [params[k] for k in capi.GPT_PARAM_NAMES]
    grads = [np.zeros_like(a) for a in pin]
    dx, loss = np.zeros_like(x), np.zeros(1, np.float32)
    ms, nodes = ctypes.c_float(0), ctypes.c_int(0)
    rc = ex.scenario_gpt_layer(DT[dtype], C, nh, B, T, V, _fp(x), targets.ctypes.data_as(ctypes.POINTER(ctypes.c_int)),
                               (FP * 20)(*map(_fp, pin)), iters, _fp(loss), (FP * 20)(*map(_fp, grads)), _fp(dx),
                               ctypes.byref(ms), ctypes.byref(nodes))
    ex.scenario_set_training(-1, ctypes.c_float(0), ctypes.c_float(0))
    if rc:
        raise SystemExit(ex.scenario_last_error().decode())
    ex.scenario_set_executor(0)
    n = B * T
    fwd = 2.0 * n * (4 * C * C + 8 * C * C + V * C) + 2 * 2.0 * T * T * (C // nh) * B * nh
    r = {"config": f"gpt layer {dtype} d768 h12 T512 B8 ff3072 V8192 fwd+bwd{' + ' + train + ' step' if train else ''} "
                   f"(block + final LayerNorm + head + loss), executor={executor}",
         "gpu_ms": round(ms.value, 3), "tflops": round(3 * fwd / ms.value / 1e9, 1), "graph_nodes": nodes.value,
         "loss": round(float(loss[0]), 4)}
    if executor & 8:
        r["kernels_per_pass"] = int(ex.scenario_recorded_kernels())
    if cpu:
        from oracle import nodes as N
        p = N.GptBlockParams(**params)
        r["cpu_ms"] = round(_cpu_timed(lambda: N.gpt_layer_forward_backward(p, x, targets, nh)), 1)
        r["cpu"] = "oracle (numpy fp32 restatement, BLAS products), 1 thread"
        # The same graph with its nodes on cpu(), in fp32 as the reference's CPU device runs it: node by node
        # through the host layer's own loops, one pass after an untimed one.
        ex.scenario_set_device(1)
        try:
            cms = ctypes.c_float(0)
            rc = ex.scenario_gpt_layer(DT["f32"], C, nh, B, T, V, _fp(x),
                                       targets.ctypes.data_as(ctypes.POINTER(ctypes.c_int)),
                                       (FP * 20)(*map(_fp, pin)), 1, _fp(loss), (FP * 20)(*map(_fp, grads)), _fp(dx),
                                       ctypes.byref(cms), ctypes.byref(nodes))
        finally:
            ex.scenario_set_device(0)
        if rc:
            raise SystemExit(ex.scenario_last_error().decode())
        r["cpu_nodes_ms"] = round(cms.value, 1)
        r["cpu_nodes"] = "the same graph on cpu() in fp32: host layer nodes, 1 thread"
    return r


def cpu_baseline(m, k, panel, dtype):
    """Blocked fp32 product of the CPU oracle, 1 thread, on an [m x k] * [k x panel] panel."""
    import numpy as np
    from oracle import cgemm
    rng = np.random.default_rng(0)
    s = 1.0 / np.sqrt(k)
    A = np.asfortranarray((rng.standard_normal((m, k), dtype=np.float32) * s))
    B = np.asfortranarray((rng.standard_normal((k, panel), dtype=np.float32) * s))
    t0 = time.perf_counter()
    cgemm.gemm(A, B, kind="f32", threads=1)
    dt = time.perf_counter() - t0
    # The same panel on the box's CPU share (OpenMP over column blocks), as a stronger courtesy line: the
    # reference itself is single-threaded, so `value` / `cores` stay the one-thread figures.
    many = max(1, min(16, cgemm.max_threads()))
    t0 = time.perf_counter()
    cgemm.gemm(A, B, kind="f32", threads=many)
    dt_many = time.perf_counter() - t0
    return {
        "value": round(2.0 * m * panel * k / dt / 1e12, 5),
        "unit": "TFLOP/s",
        "cores": 1,
        "kind": "port",
        "sample": f"oracle_gemm_f32 (blocked fp32, 1 thread, as the reference's single-threaded Eigen build) "
                  f"on a {m}x{k} * {k}x{panel} column panel of the same product, {dt:.1f} s; "
                  f"host has {os.cpu_count()} logical cores",
        "all_cores": {"value": round(2.0 * m * panel * k / dt_many / 1e12, 5), "cores": many,
                      "seconds": round(dt_many, 2)},
    }


def measured_traffic(dtype, layout, m, n, k):
    """(bytes per launch, source) from profiles/hbm_traffic.txt, or (None, None)."""
    if not TRAFFIC_FILE.exists():
        return None, None
    for line in TRAFFIC_FILE.read_text().splitlines():
        f = line.split()
        if len(f) >= 7 and not line.startswith("#") and f[:5] == [dtype, layout, str(m), str(n), str(k)]:
            return int(f[5]), f[6]
    return None, None


def other_configs(h, cpu):
    """The other configurations of the build target, outside the headline's timed region.  Graph level (GPU
    ms per fwd+bwd pass through the frozen level executor, algorithmic GB/s, kernel launches per pass counted
    in a recording of the pass, the CPU oracle on one thread beside them): min-GPT layer, MLP, autobatched
    LSTM.  Kernel level: the six attention products, the skinny shapes M = K = 4096 and two more squares of
    the GEMM sweep, each against the roofline that bounds it."""
    out = {}
    # Kernel-level figures first, while the clocks the headline product raised are still up: the CPU legs of
    # the graph-level configurations below leave the device idle for seconds.
    out["attention"] = {r["config"].split("batch 128 ")[1]: {"us": round(r["gpu_ms"] * 1e3, 2), "gbs": r["gbs"],
                                                             "frac_hbm": r["frac_hbm"], "tflops": r["tflops"]}
                        for r in bench_attention(h, 200, 20, False)}
    skinny = {}
    for dt in ("f32", "f16"):
        for nn in (1, 16, 64):
            ms = time_product(h, dt, "NN", 4096, nn, 4096, 200, 20)
            by = ESIZE[dt] * (4096 * 4096 + 4096 * nn + 4096 * nn)
            tf = 2.0 * 4096 * nn * 4096 / ms / 1e9
            skinny[f"{dt}_n{nn}"] = {"us": round(ms * 1e3, 2), "gbs": round(by / ms / 1e6, 1),
                                     "frac_hbm": round(by / ms / 1e6 / PEAK_HBM_GBS, 4),
                                     "frac_mfma": round(tf / PEAK_TFLOPS[dt], 4)}
    out["skinny_m4096_k4096"] = skinny
    squares = {}
    for size, steps in ((4096, 100), (2048, 200)):
        ms = time_product(h, "f16", "NN", size, size, size, steps, 20)
        tf = 2.0 * size ** 3 / ms / 1e9
        squares[f"f16_NN_{size}"] = {"us": round(ms * 1e3, 2), "tflops": round(tf, 1),
                                     "frac_mfma": round(tf / PEAK_TFLOPS["f16"], 4)}
    out["squares"] = squares
    g = bench_gpt(30, cpu, executor=6)
    out["gpt_ms"], out["gpt_tflops"] = g["gpu_ms"], g["tflops"]
    if cpu:
        out["gpt_cpu_ms"] = g["cpu_ms"]
        out["gpt_cpu_nodes_ms"] = g["cpu_nodes_ms"]
    out["gpt_kernels_per_pass"] = bench_gpt(2, False, executor=14)["kernels_per_pass"]
    r = bench_mlp(100, cpu, executor=6)
    out["mlp_ms"], out["mlp_gbs"] = r["gpu_ms"], r["gbs"]
    if cpu:
        out["mlp_cpu_ms"] = r["cpu_ms"]
        out["mlp_cpu_nodes_ms"] = r["cpu_nodes_ms"]
    out["mlp_kernels_per_pass"] = bench_mlp(2, False, executor=14)["kernels_per_pass"]
    r = bench_lstm(10, cpu, mode=23, gather=True)
    out["lstm_ms"], out["lstm_gbs"] = r["gpu_ms"], r["gbs"]
    out["lstm_table_launches_per_pass"] = r["table_launches_per_pass"]
    if cpu:
        out["lstm_cpu_ms"] = r["cpu_ms"]
        out["lstm_cpu_nodes_ms"] = r["cpu_nodes_ms"]
    out["lstm_kernels_per_pass"] = bench_lstm(2, False, mode=31, gather=True)["kernels_per_pass"]
    out["note"] = ("fwd+bwd per pass: min-GPT layer bf16 (d768 h12 T512 B8 ff3072 V8192), MLP fp32 b64 784-512-512-10, "
                   "autobatched LSTM fp32 256 seqs; gbs = algorithmic bytes of the pass's products per second; "
                   "kernels_per_pass = kernel nodes of the pass recorded as a device graph; attention = fp16 batch 128 "
                   "products, skinny = M = K = 4096 NN with the split-K fold included, against 8 TB/s; squares "
                   "against 2.5 PFLOP/s; cpu = numpy fp32 oracle on 1 thread; gpt_cpu_nodes_ms / mlp_cpu_nodes_ms / "
                   "lstm_cpu_nodes_ms = the same graph with its nodes on cpu() (the host layer's own fp32 loops and "
                   "packed product, node by node, 1 thread)")
    return out


def main():
    a = parse_args()
    if a.gpus != 1:
        raise SystemExit("bench.py: this build measures one GPU only; run with --gpus 1 "
                         "(sharding over several GPUs is a design note of this build, not code)")
    h = Harness()
    m = k = a.size
    n = a.n or a.size

    if a.workload == "copy":
        # One [size x size] copy per step through ginn_hip_copy_2d: reads and writes
        # size * size * esize bytes each; used to scale FETCH_SIZE / WRITE_SIZE.
        t = h.torch
        src = t.ones(a.size, a.size, device="cuda", dtype=h.tdtype(a.dtype))
        dst = t.zeros_like(src)
        t.cuda.synchronize()
        for _ in range(a.warmup + a.steps):
            h.lib.call("ginn_hip_copy_2d", h.ctx, DT[a.dtype], a.size, a.size, c_void_p(src.data_ptr()), a.size,
                       c_void_p(dst.data_ptr()), a.size, 0)
        h.lib.call("ginn_hip_sync", h.ctx)
        print(json.dumps({"workload": "copy", "bytes_read_per_launch": a.size * a.size * ESIZE[a.dtype],
                          "bytes_written_per_launch": a.size * a.size * ESIZE[a.dtype]}))
        return

    if a.workload == "ragged":
        for r in bench_ragged(h, max(1, a.steps), a.warmup):
            print(json.dumps(r), flush=True)
        return

    if a.workload == "skinny":
        for r in bench_skinny(h, max(1, a.steps), a.warmup):
            print(json.dumps(r), flush=True)
        return

    if a.workload in ("configs", "mlp", "lstm", "attention", "gpt", "update"):
        cpu = not a.no_cpu
        iters = max(1, a.steps)
        out = []
        if a.workload in ("configs", "mlp"):
            out.append(bench_mlp(iters, cpu, executor=14))
            out.append(bench_mlp(iters, False, executor=6))
            out.append(bench_mlp(iters, False, executor=0))
        if a.workload in ("configs", "lstm"):
            out.append(bench_lstm(max(1, iters // 5), cpu, mode=31, gather=True))
            out.append(bench_lstm(max(1, iters // 5), False, mode=23, gather=True))
            out.append(bench_lstm(max(1, iters // 5), False, mode=23))
            out.append(bench_lstm(max(1, iters // 5), False, mode=15, gather=True))
            out.append(bench_lstm(max(1, iters // 5), False, mode=7, gather=True))
            out.append(bench_lstm(max(1, iters // 5), False, mode=15))
            out.append(bench_lstm(max(1, iters // 5), False, mode=7))
            out.append(bench_lstm(max(1, iters // 10), False, mode=3))
        if a.workload == "configs":
            out.append(bench_lstm(max(1, iters // 20), False, mode=1))
            out.append(bench_lstm(max(1, iters // 20), False, mode=0))
        if a.workload in ("configs", "attention"):
            out.extend(bench_attention(h, iters, a.warmup, cpu, store_floor=a.workload == "attention"))
        if a.workload in ("configs", "update"):
            out.extend(bench_update(h, iters, a.warmup, cpu))
        if a.workload in ("configs", "gpt"):
            out.append(bench_gpt(max(1, iters // 5), cpu, executor=14))
            out.append(bench_gpt(max(1, iters // 5), False, executor=6))
            out.append(bench_gpt(max(1, iters // 5), False, executor=6, train="adam"))
            out.append(bench_gpt(max(1, iters // 5), False, executor=0))
        for r in out:
            print(json.dumps(r), flush=True)
        if a.report:
            Path(a.report).parent.mkdir(parents=True, exist_ok=True)
            Path(a.report).write_text(json.dumps(out, indent=1))
        return

    results = []
    if a.workload == "sweep":
        shapes = []
        for dt in ("f32", "f16", "bf16"):
            for lay in ("NN", "NT", "TN"):
                for s in (512, 1024, 2048, 4096, 8192):
                    shapes.append((dt, lay, s, s, s))
            for nn in (1, 16, 64):
                shapes.append((dt, "NN", 4096, nn, 4096))
        for dt, lay, mm, nn, kk in shapes:
            steps = max(5, min(a.steps, int(2e12 / (2.0 * mm * nn * kk)) + 5))
            wall, ms, _ = h.time_gemm(dt, lay, mm, nn, kk, steps, max(2, a.warmup // 2))
            fl = 2.0 * mm * nn * kk
            by = ESIZE[dt] * (mm * kk + kk * nn + mm * nn)
            r = {"dtype": dt, "layout": lay, "m": mm, "n": nn, "k": kk, "ms": round(ms, 5),
                 "tflops": round(fl / ms / 1e9, 3), "frac_mfma": round(fl / ms / 1e9 / PEAK_TFLOPS[dt], 4),
                 "gbs": round(by / ms / 1e6, 2), "frac_hbm": round(by / ms / 1e6 / PEAK_HBM_GBS, 4)}
            results.append(r)
            print(json.dumps(r), file=sys.stderr, flush=True)
        if a.report:
            Path(a.report).parent.mkdir(parents=True, exist_ok=True)
            Path(a.report).write_text(json.dumps(results, indent=1))

    wall, kernel_ms, _ = h.time_gemm(a.dtype, a.layout, m, n, k, a.steps, a.warmup, a.beta,
                                     ramp_seconds=0.0 if a.no_ramp else RAMP_SECONDS)
    traffic, traffic_source = measured_traffic(a.dtype, a.layout, m, n, k) if a.beta == 0 else (None, None)
    flops = 2.0 * m * n * k
    value = flops * a.steps / wall / 1e12
    achieved = flops / (kernel_ms * 1e-3) / 1e12
    line = {
        "metric": f"{a.dtype} ginn::gemm M=N=K={a.size} TFLOP/s" if n == a.size else
                  f"{a.dtype} ginn::gemm M=K={a.size} N={n} TFLOP/s",
        "value": round(value, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": a.steps,
        "warmup": a.warmup,
        "ramp_launches": h.ramp_launches,
        "ms_per_step": round(wall / a.steps * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": a.dtype,
        "data": "synthetic",
        "config": {"workload": f"GEMM sweep via ginn::prod: {a.dtype} (fp32 accumulate) {a.layout} "
                               f"column-major {m}x{k} * {k}x{n}, entries N(0,1)/sqrt(K)",
                   "entry_point": "ginn_hip_gemm", "beta": a.beta},
        "roofline": {
            "bound": "mfma",
            "achieved": round(achieved, 2),
            "peak": PEAK_TFLOPS[a.dtype],
            "unit": "TFLOP/s",
            "frac": round(achieved / PEAK_TFLOPS[a.dtype], 4),
            "traffic": traffic,
            "traffic_source": traffic_source,
            "kernel_ms": round(kernel_ms, 4),
        },
    }
    # A shape with fewer flops per algorithmic byte than the part has per byte of HBM bandwidth (narrow
    # right-hand sides) is bound by memory: its roofline is algorithmic bytes per second against 8 TB/s.
    algo_bytes = ESIZE[a.dtype] * (m * k + k * n + m * n * (2 if a.beta != 0 else 1))
    if flops / algo_bytes < PEAK_TFLOPS[a.dtype] * 1e12 / (PEAK_HBM_GBS * 1e9):
        gbs = algo_bytes / (kernel_ms * 1e-3) / 1e9
        line["roofline"].update({"bound": "hbm", "achieved": round(gbs, 1), "peak": PEAK_HBM_GBS, "unit": "GB/s",
                                 "frac": round(gbs / PEAK_HBM_GBS, 4)})
    # The other configurations right behind the headline product (their kernel-level part wants the clocks it
    # raised); the CPU baseline, seconds of host work with the device idle, last.  The keys keep their order.
    configs = None if a.no_configs else other_configs(h, not a.no_cpu)
    if not a.no_cpu:
        line["cpu_baseline"] = cpu_baseline(m, k, min(a.cpu_panel, n), a.dtype)
    if configs is not None:
        line["configs"] = configs
    print(json.dumps(line), flush=True)


if __name__ == "__main__":
    main()
