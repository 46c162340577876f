"""Device memory behind the C ABI: the block cache of ginn_hip_malloc /
ginn_hip_free (in place of one cudaMalloc / cudaFree per temporary tensor,
ginn/dev.h:158-175), the byte-exact arena (ginn/dev.h:214-254), fills and
copies at any alignment."""
import ctypes
from ctypes import byref, c_size_t, c_void_p

import numpy as np
import pytest

from ginn_amd import capi

pytestmark = pytest.mark.gpu


@pytest.fixture()
def ctx():
    lib = capi.load()
    c = lib.ctx_create(0)
    yield lib, c
    lib.call("ginn_hip_ctx_destroy", c)


def stats(lib, c):
    cached, blocks = c_size_t(0), c_size_t(0)
    lib.call("ginn_hip_pool_stats", c, byref(cached), byref(blocks))
    return cached.value, blocks.value


def test_released_blocks_are_reused(ctx):
    lib, c = ctx
    p, q = c_void_p(), c_void_p()
    lib.call("ginn_hip_malloc", c, 1000, byref(p))
    assert stats(lib, c) == (0, 1)
    lib.call("ginn_hip_free", c, p)
    assert stats(lib, c) == (1024, 1)  # held, rounded to the block size
    lib.call("ginn_hip_malloc", c, 700, byref(q))  # same block size: no driver call
    assert q.value == p.value and stats(lib, c) == (0, 1)
    r = c_void_p()
    lib.call("ginn_hip_malloc", c, 5 << 20, byref(r))  # above 2 MiB: multiples of 2 MiB
    lib.call("ginn_hip_free", c, r)
    assert stats(lib, c) == (6 << 20, 2)
    lib.call("ginn_hip_pool_trim", c)
    assert stats(lib, c) == (0, 1)
    lib.call("ginn_hip_free", c, q)
    # switched off: malloc / free go to the driver
    lib.call("ginn_hip_pool_configure", c, 0, 0)
    assert stats(lib, c) == (0, 0)
    lib.call("ginn_hip_malloc", c, 1000, byref(p))
    lib.call("ginn_hip_free", c, p)
    assert stats(lib, c) == (0, 0)
    # a bound: what does not fit goes back to the driver
    lib.call("ginn_hip_pool_configure", c, 1, 4096)
    lib.call("ginn_hip_malloc", c, 8192, byref(p))
    lib.call("ginn_hip_free", c, p)
    assert stats(lib, c) == (0, 0)


def test_reuse_is_ordered_on_the_stream(ctx):
    """A block is released while a copy out of it is still enqueued, handed out
    again and overwritten: the copy sees the old contents (one stream)."""
    lib, c = ctx
    n = 1 << 20
    a, b, keep = c_void_p(), c_void_p(), c_void_p()
    lib.call("ginn_hip_malloc", c, 4 * n, byref(a))
    lib.call("ginn_hip_malloc", c, 4 * n, byref(keep))
    lib.call("ginn_hip_fill", c, capi.F32, a, n, 3.0)
    lib.call("ginn_hip_memcpy_d2d", c, keep, a, 4 * n)  # enqueued, not waited for
    lib.call("ginn_hip_free", c, a)
    lib.call("ginn_hip_malloc", c, 4 * n, byref(b))
    assert b.value == a.value
    lib.call("ginn_hip_fill", c, capi.F32, b, n, 7.0)
    host = np.zeros(n, np.float32)
    lib.call("ginn_hip_memcpy_d2h", c, host.ctypes.data_as(c_void_p), keep, 4 * n)
    assert (host == 3.0).all()
    lib.call("ginn_hip_memcpy_d2h", c, host.ctypes.data_as(c_void_p), b, 4 * n)
    assert (host == 7.0).all()


def test_arena_is_byte_exact_and_fills_work_at_any_alignment(ctx):
    lib, c = ctx
    arena = c_void_p()
    lib.call("ginn_hip_arena_create", c, 1000, byref(arena))
    used, p1, p2, p3 = c_size_t(0), c_void_p(), c_void_p(), c_void_p()
    lib.call("ginn_hip_arena_alloc", arena, 6, byref(p1))
    lib.call("ginn_hip_arena_alloc", arena, 10, byref(p2))
    lib.call("ginn_hip_arena_used", arena, byref(used))
    assert used.value == 16 and p2.value == p1.value + 6  # blocks back to back (ginn/dev.h:236-248)
    # fp16 fill and byte fill of a block that starts 6 bytes into the slab
    lib.call("ginn_hip_fill", c, capi.F16, p2, 5, 1.5)
    host = np.zeros(5, np.float16)
    lib.call("ginn_hip_memcpy_d2h", c, host.ctypes.data_as(c_void_p), p2, 10)
    assert (host == 1.5).all()
    lib.call("ginn_hip_memset", c, p1, 0xAB, 6)
    raw = np.zeros(16, np.uint8)
    lib.call("ginn_hip_memcpy_d2h", c, raw.ctypes.data_as(c_void_p), p1, 16)
    assert (raw[:6] == 0xAB).all() and (raw[6:].view(np.float16) == 1.5).all()
    # strict '<': 984 more bytes would fill the slab exactly and are refused, 983 fit
    with pytest.raises(capi.GinnHipError, match="out of memory"):
        lib.call("ginn_hip_arena_alloc", arena, 984, byref(p3))
    lib.call("ginn_hip_arena_alloc", arena, 983, byref(p3))
    lib.call("ginn_hip_arena_set_alignment", arena, 64)
    lib.call("ginn_hip_arena_clear", arena)
    lib.call("ginn_hip_arena_alloc", arena, 3, byref(p1))
    lib.call("ginn_hip_arena_alloc", arena, 3, byref(p2))
    lib.call("ginn_hip_arena_used", arena, byref(used))
    assert p2.value == p1.value + 64 and used.value == 67
    lib.call("ginn_hip_arena_destroy", arena)


def test_a_context_waits_for_another(ctx):
    """ginn_hip_ctx_wait_for: what is enqueued on the waiter afterwards sees everything the signaler had
    enqueued before (no host wait in between); one stream needs no event; while a device graph is being
    recorded nothing is ordered and the caller is told so."""
    from ctypes import c_int
    lib, a = ctx
    b = lib.ctx_create(0)
    try:
        n = 1 << 24
        buf, out = c_void_p(), c_void_p()
        lib.call("ginn_hip_malloc", a, 4 * n, byref(buf))
        lib.call("ginn_hip_malloc", a, 4 * n, byref(out))
        lib.call("ginn_hip_fill", a, capi.F32, out, n, -1.0)
        lib.call("ginn_hip_sync", a)
        for i in range(40):  # a queue of fills on a; the last one counts
            lib.call("ginn_hip_fill", a, capi.F32, buf, n, float(i))
        ordered = c_int(-1)
        lib.call("ginn_hip_ctx_wait_for", b, a, byref(ordered))
        assert ordered.value == 1
        lib.call("ginn_hip_memcpy_d2d", b, out, buf, 4 * n)
        host = np.zeros(n, np.float32)
        lib.call("ginn_hip_memcpy_d2h", b, host.ctypes.data_as(c_void_p), out, 4 * n)
        assert (host == 39.0).all()
        lib.call("ginn_hip_ctx_wait_for", a, a, byref(ordered))
        assert ordered.value == 1
        lib.call("ginn_hip_capture_begin", a)
        try:
            lib.call("ginn_hip_fill", a, capi.F32, buf, n, 5.0)
            lib.call("ginn_hip_ctx_wait_for", b, a, byref(ordered))
            assert ordered.value == 0
        finally:
            graph = c_void_p()
            lib.call("ginn_hip_capture_end", a, byref(graph))
            lib.call("ginn_hip_graph_destroy", graph)
        with pytest.raises(capi.GinnHipError, match="NULL"):
            lib.call("ginn_hip_ctx_wait_for", b, None, byref(ordered))
        lib.call("ginn_hip_free", a, buf)
        lib.call("ginn_hip_free", a, out)
    finally:
        lib.call("ginn_hip_ctx_destroy", b)
