"""ginn_hip_gemm_noalloc (the product entry point that allocates nothing)
against ginn_hip_gemm on the same operands, through the C ABI: two calls in a
row on one GPU, the second on a smaller input, so that whatever the first call
left in the per-GPU scratch array is there when the second runs; then the
refusal of an output beyond the array's limit."""
import ctypes

import numpy as np
import pytest

from conftest import rel_fro
from ginn_amd import capi

pytestmark = pytest.mark.gpu

# (dtype, m, n, k): shapes whose kernels keep split-K partial sums in scratch memory,
# first the larger, then a smaller one.
CASES = [
    (capi.F32, [(4096, 16, 4096), (1024, 9, 2048)]),     # matrix-core skinny kernel, K split over blocks
    (capi.F32, [(4096, 1, 4096), (512, 64, 784)]),       # vector skinny kernel; generic kernel with split-K
    (capi.F16, [(4096, 4, 8192), (2048, 1, 4096)]),      # 16-bit skinny kernel
    (capi.BF16, [(768, 768, 4096), (256, 128, 2048)]),   # 128 x 128 family with split-K
    (capi.F16, [(1000, 1000, 1000), (200, 136, 72)]),    # masked tile edges (no copies, no cuts)
]


@pytest.mark.parametrize("dt,shapes", CASES)
def test_noalloc_matches_gemm_on_two_calls(dt, shapes):
    from gpu_util import TIGHT, TOL, Dev, round_to
    dev = Dev()
    torch = dev.torch
    stream = torch.cuda.current_stream().cuda_stream
    rng = np.random.default_rng(shapes[0][0] + shapes[0][1])
    try:
        for m, n, k in shapes:
            a = round_to(rng.standard_normal((m, k)) / np.sqrt(k), dt)
            b = round_to(rng.standard_normal((k, n)), dt)
            c0 = round_to(rng.standard_normal((m, n)), dt)
            ba, pa, lda = dev.put(a, dt)
            bb, pb, ldb = dev.put(b, dt)
            for beta in (0.0, 1.0):
                b1, p1, ld1 = dev.put(c0, dt)
                b2, p2, ld2 = dev.put(c0, dt)
                dev.gemm(dt, 0, 0, m, n, k, pa, lda, pb, ldb, beta, p1, ld1)
                dev.lib.call("ginn_hip_gemm_noalloc", 0, ctypes.c_void_p(stream), dt, 0, 0, m, n, k,
                             ctypes.c_void_p(pa), lda, ctypes.c_void_p(pb), ldb, beta, ctypes.c_void_p(p2), ld2)
                dev.sync()
                ref, got = dev.get(b1, (m, n)), dev.get(b2, (m, n))
                want = a.astype(np.float64) @ b.astype(np.float64) + beta * c0.astype(np.float64)
                assert rel_fro(ref, want) <= TOL[dt]
                assert rel_fro(got, want) <= TOL[dt]
                # the two entry points run the same kernels; only the number of K splits may differ
                assert rel_fro(got, ref) <= TIGHT[dt]
    finally:
        dev.close()


def test_noalloc_refuses_outputs_beyond_the_scratch_limit():
    from gpu_util import Dev
    dev = Dev()
    try:
        t = dev.torch.zeros(16, device="cuda")
        p = ctypes.c_void_p(t.data_ptr())
        rc = dev.lib.cdll.ginn_hip_gemm_noalloc(0, None, capi.F32, 0, 0, 2048, 2048, 8, p, 2048, p, 8, 0.0, p, 2048)
        assert rc != 0
        msg = dev.lib.last_error()
        assert "exceeds" in msg and "scratch" in msg, msg
        # at the limit the size check passes (m * n = 2 097 152): the next check to fail is another one
        rc = dev.lib.cdll.ginn_hip_gemm_noalloc(0, None, capi.F32, 0, 0, 2048, 1024, 8, None, 2048, p, 8, 0.0, p, 2048)
        assert rc != 0 and "exceeds" not in dev.lib.last_error()
    finally:
        dev.close()
