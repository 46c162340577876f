"""ctypes declarations of the C ABI in ``include/ginn_hip.h``.

Loading fails loudly (``GinnHipError``) when the library has not been built;
there is no fallback of any kind.
"""
from __future__ import annotations

import ctypes
import importlib.util
from ctypes import (POINTER, byref, c_char_p, c_float, c_int, c_longlong, c_ulonglong,
                    c_size_t, c_void_p)
from pathlib import Path

PKG = Path(__file__).resolve().parent
LIB_PATH = PKG / "lib" / "libginn_hip.so"

F32, F16, BF16 = 0, 1, 2
OP_N, OP_T = 0, 1
(ACT_IDENTITY, ACT_TANH, ACT_RELU, ACT_SIGMOID, ACT_GELU, ACT_GELU2,
 ACT_SOFTMAX, ACT_LOG, ACT_SQRT) = range(9)

# name -> (restype, argtypes); mirrors include/ginn_hip.h one to one.
# Order in which scenario_gpt_layer (ginn_amd/examples/configs.cpp) takes the 20 parameters of one
# decoder layer + final LayerNorm + vocabulary head (examples/min-gpt.cu.cpp:93-163, 227-260).
GPT_PARAM_NAMES = ["ln1_g", "ln1_b", "Wk", "bk", "Wq", "bq", "Wv", "bv", "Wp", "bp", "ln2_g", "ln2_b", "W1", "b1",
                   "W2", "b2", "lnf_g", "lnf_b", "Wh", "bh"]

PROTOTYPES = {
    "ginn_hip_last_error": (c_char_p, []),
    "ginn_hip_version": (c_char_p, []),
    "ginn_hip_device_count": (c_int, [POINTER(c_int)]),
    "ginn_hip_ctx_create": (c_int, [c_int, c_size_t, POINTER(c_void_p)]),
    "ginn_hip_ctx_create_on_stream": (c_int, [c_int, c_void_p, c_size_t, POINTER(c_void_p)]),
    "ginn_hip_ctx_destroy": (c_int, [c_void_p]),
    "ginn_hip_ctx_device": (c_int, [c_void_p, POINTER(c_int)]),
    "ginn_hip_ctx_stream": (c_int, [c_void_p, POINTER(c_void_p)]),
    "ginn_hip_sync": (c_int, [c_void_p]),
    "ginn_hip_malloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "ginn_hip_free": (c_int, [c_void_p, c_void_p]),
    "ginn_hip_pool_configure": (c_int, [c_void_p, c_int, c_size_t]),
    "ginn_hip_pool_trim": (c_int, [c_void_p]),
    "ginn_hip_gemm_temp_budget": (c_int, [c_void_p, c_size_t]),
    "ginn_hip_pool_stats": (c_int, [c_void_p, POINTER(c_size_t), POINTER(c_size_t)]),
    "ginn_hip_memcpy_h2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "ginn_hip_memcpy_d2h": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "ginn_hip_memcpy_d2d": (c_int, [c_void_p, c_void_p, c_void_p, c_size_t]),
    "ginn_hip_memset": (c_int, [c_void_p, c_void_p, c_int, c_size_t]),
    "ginn_hip_arena_create": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "ginn_hip_arena_destroy": (c_int, [c_void_p]),
    "ginn_hip_arena_alloc": (c_int, [c_void_p, c_size_t, POINTER(c_void_p)]),
    "ginn_hip_arena_clear": (c_int, [c_void_p]),
    "ginn_hip_arena_set_alignment": (c_int, [c_void_p, c_size_t]),
    "ginn_hip_arena_used": (c_int, [c_void_p, POINTER(c_size_t)]),
    "ginn_hip_arena_size": (c_int, [c_void_p, POINTER(c_size_t)]),
    "ginn_hip_gemm": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                              c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int]),
    "ginn_hip_gemm_noalloc": (c_int, [c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                      c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_int]),
    "ginn_hip_gemm_strided_batched": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                              c_void_p, c_int, c_longlong, c_void_p, c_int, c_longlong,
                                              c_float, c_void_p, c_int, c_longlong, c_int]),
    "ginn_hip_gemm_strided_batched2": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                               c_void_p, c_int, c_longlong, c_longlong, c_void_p, c_int, c_longlong,
                                               c_longlong, c_float, c_void_p, c_int, c_longlong, c_longlong, c_int,
                                               c_int]),
    "ginn_hip_gemm_grouped": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int,
                                      POINTER(c_void_p), POINTER(c_int), POINTER(c_int), c_float,
                                      POINTER(c_void_p), POINTER(c_int)]),
    "ginn_hip_gemm_gathered": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                       c_void_p, c_int, c_void_p, c_float, c_void_p, c_int, c_void_p, c_int]),
    "ginn_hip_gemm_outer_sum": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p,
                                        c_int, c_int]),
    "ginn_hip_col_dot_batched": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p]),
    "ginn_hip_affine_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, POINTER(c_void_p),
                                    POINTER(c_void_p), POINTER(c_int), c_void_p, c_void_p, c_void_p]),
    "ginn_hip_affine_bwd_pre": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_void_p]),
    "ginn_hip_nonlin_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ginn_hip_nonlin_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                    c_void_p, c_int]),
    "ginn_hip_fill": (c_int, [c_void_p, c_int, c_void_p, c_size_t, c_float]),
    "ginn_hip_copy_2d": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_int]),
    "ginn_hip_add_n": (c_int, [c_void_p, c_int, c_size_t, c_int, POINTER(c_void_p), c_void_p, c_int]),
    "ginn_hip_cwise_prod": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_int]),
    "ginn_hip_scale_shift": (c_int, [c_void_p, c_int, c_size_t, c_float, c_float, c_void_p, c_void_p, c_int]),
    "ginn_hip_col_broadcast": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ginn_hip_row_sum": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "ginn_hip_sum_all": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_float, c_void_p]),
    "ginn_hip_add_scalar_bcast": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_float, c_void_p]),
    "ginn_hip_pick_nls_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick_nls_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick_nls_fwd_stats": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick_nls_bwd_stats": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_int]),
    "ginn_hip_pick_nls_bwd_assign": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_layernorm_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p]),
    "ginn_hip_layernorm_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_cwise_prod_add_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float,
                                            c_int, c_void_p]),
    "ginn_hip_cwise_prod_add_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float,
                                            c_int, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_cwise_prod_add_bwd_assign": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_float,
                                            c_int, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_layernorm_affine_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p,
                                              c_float, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_layernorm_affine_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                              c_float, c_void_p, c_int, c_void_p, c_void_p]),
    "ginn_hip_permute": (c_int, [c_void_p, c_int, c_int, POINTER(c_longlong), POINTER(c_int), c_void_p, c_void_p,
                                 c_int]),
    "ginn_hip_mask_fill": (c_int, [c_void_p, c_int, c_size_t, c_size_t, c_void_p, c_float, c_void_p]),
    "ginn_hip_scaled_masked_softmax_fwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p,
                                                   c_size_t, c_float, c_void_p]),
    "ginn_hip_scaled_masked_softmax_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float,
                                                   c_void_p, c_size_t, c_void_p]),
    "ginn_hip_upper_tri": (c_int, [c_void_p, c_int, c_int, c_void_p]),
    "ginn_hip_defer_folds": (c_int, [c_void_p, c_int]),
    "ginn_hip_flush_folds": (c_int, [c_void_p]),
    "ginn_hip_pending_folds": (c_int, [c_void_p, POINTER(c_int)]),
    "ginn_hip_layernorm_bwd_assign": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_elementwise": (c_int, [c_void_p, c_int, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p, c_int]),
    "ginn_hip_fill_uniform": (c_int, [c_void_p, c_int, c_size_t, c_ulonglong, c_float, c_float, c_void_p]),
    "ginn_hip_dropout_mask": (c_int, [c_void_p, c_size_t, c_float, c_ulonglong, c_void_p]),
    "ginn_hip_mask_scale": (c_int, [c_void_p, c_int, c_size_t, c_float, c_void_p, c_void_p, c_void_p, c_int]),
    "ginn_hip_select": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p]),
    "ginn_hip_select_bwd": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_int, c_void_p, c_void_p, c_int]),
    "ginn_hip_mask_select": (c_int, [c_void_p, c_int, c_size_t, c_size_t, c_void_p, c_float, c_void_p, c_void_p, c_int]),
    "ginn_hip_less_than": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick_bwd": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_float, c_void_p]),
    "ginn_hip_pick_nlsig_fwd": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_pick_nlsig_bwd": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_axis_sum": (c_int, [c_void_p, c_int, c_int, POINTER(c_longlong), POINTER(c_int), c_void_p, c_void_p]),
    "ginn_hip_axis_sum_bwd": (c_int, [c_void_p, c_int, c_int, POINTER(c_longlong), POINTER(c_int), c_void_p, c_void_p]),
    "ginn_hip_variance_fwd": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_variance_bwd": (c_int, [c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_stack": (c_int, [c_void_p, c_int, c_size_t, c_size_t, c_void_p, c_void_p]),
    "ginn_hip_stack_bwd": (c_int, [c_void_p, c_int, c_size_t, c_size_t, c_void_p, c_void_p]),
    "ginn_hip_argmax": (c_int, [c_void_p, c_int, c_size_t, c_size_t, c_size_t, c_void_p, c_void_p]),
    "ginn_hip_row_broadcast": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ginn_hip_col_sum": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_int]),
    "ginn_hip_multi_apply": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_float, c_size_t, c_int, c_void_p,
                                     c_void_p, c_void_p, c_void_p]),
    "ginn_hip_multi_mixed": (c_int, [c_void_p, c_int, c_void_p, c_size_t]),
    "ginn_hip_multi_chain": (c_int, [c_void_p, c_int, c_void_p, c_void_p]),
    "ginn_hip_ctx_wait_for": (c_int, [c_void_p, c_void_p, POINTER(c_int)]),
    "ginn_hip_multi_reduce": (c_int, [c_void_p, c_int, c_size_t, c_int, c_void_p, c_void_p, c_int]),
    "ginn_hip_multi_zero": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_size_t]),
    "ginn_hip_update": (c_int, [c_void_p, c_void_p, c_int, c_size_t, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ginn_hip_multi_update": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_size_t]),
    "ginn_hip_capture_begin": (c_int, [c_void_p]),
    "ginn_hip_capture_end": (c_int, [c_void_p, POINTER(c_void_p)]),
    "ginn_hip_graph_launch": (c_int, [c_void_p]),
    "ginn_hip_graph_kernel_count": (c_int, [c_void_p, POINTER(c_size_t)]),
    "ginn_hip_graph_destroy": (c_int, [c_void_p]),
    "ginn_hip_event_record": (c_int, [c_void_p, c_int]),
    "ginn_hip_event_elapsed_ms": (c_int, [c_void_p, c_int, c_int, POINTER(c_float)]),
}


class UpdateRule(ctypes.Structure):
    """ginn_hip_update_rule."""
    _fields_ = [("kind", c_int), ("lr", c_float), ("clip", c_float), ("beta1", c_float),
                ("one_minus_beta1", c_float), ("beta2", c_float), ("one_minus_beta2", c_float),
                ("step", c_float), ("vscale", c_float), ("eps", c_float)]


class UpdateOp(ctypes.Structure):
    """ginn_hip_update_op."""
    _fields_ = [("w", c_void_p), ("g", c_void_p), ("m", c_void_p), ("v", c_void_p), ("n", c_size_t),
                ("dtype", c_int), ("reserved", c_int)]


UPDATE_SGD, UPDATE_ADAM = 0, 1


class GinnHipError(RuntimeError):
    """A C-ABI call returned a non-zero status (message from ginn_hip_last_error)."""


class Library:
    """The loaded shared library with typed entry points.

    ``lib.call("ginn_hip_gemm", ...)`` raises GinnHipError on a non-zero status.
    """

    def __init__(self, path: Path = LIB_PATH):
        if not Path(path).exists():
            raise GinnHipError(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)")
        self.path = Path(path)
        # A process must hold ONE HIP runtime: device pointers and streams of one
        # copy mean nothing to another.  PyTorch wheels bundle their own copy and
        # ask for it by file name, so it is loaded beside the system's if that is
        # already there (and then finds no GPU); loaded first, it satisfies this
        # library's libamdhip64.so.7 by soname and both share it.
        if importlib.util.find_spec("torch") is not None:
            import torch  # noqa: F401
        self.cdll = ctypes.CDLL(str(path))
        for name, (res, args) in PROTOTYPES.items():
            fn = getattr(self.cdll, name)  # AttributeError if the symbol is missing
            fn.restype = res
            fn.argtypes = args

    def last_error(self) -> str:
        return self.cdll.ginn_hip_last_error().decode()

    def call(self, name: str, *args):
        rc = getattr(self.cdll, name)(*args)
        if rc != 0:
            raise GinnHipError(f"{name} -> {rc}: {self.last_error()}")
        return rc

    # -- small conveniences used by tests and bench ---------------------------
    def device_count(self) -> int:
        n = c_int(0)
        self.call("ginn_hip_device_count", byref(n))
        return n.value

    def ctx_create(self, device: int = 0, workspace_bytes: int = 0) -> c_void_p:
        ctx = c_void_p()
        self.call("ginn_hip_ctx_create", device, workspace_bytes, byref(ctx))
        return ctx

    def ctx_create_on_stream(self, device: int, stream: int, workspace_bytes: int = 0) -> c_void_p:
        ctx = c_void_p()
        self.call("ginn_hip_ctx_create_on_stream", device, c_void_p(stream), workspace_bytes, byref(ctx))
        return ctx


_library = None


def load() -> Library:
    """Returns the process-wide Library, loading it on first use."""
    global _library
    if _library is None:
        _library = Library()
    return _library
