"""ctypes binding of the C-ABI library `libmlk.so` (declared in include/mlk.h).

The library is loaded from this directory only.  There is no fallback: if the
library is missing or an entry point fails, a RuntimeError is raised.
"""
import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmlk.so")

c_void_p, c_int, c_int64, c_float, c_size_t = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float,
                                               ctypes.c_size_t)

# name -> (restype, argtypes); mirrors include/mlk.h one to one
SIGNATURES = {
    "mlk_version": (c_int, []),
    "mlk_last_error": (ctypes.c_char_p, []),
    "mlk_set_tunable": (None, [c_int, c_int]),
    "mlk_moe_set_tile_path": (None, [c_int]),
    "mlk_pack_layout_a": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "mlk_unpack_layout_a": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_void_p]),
    "mlk_layout_b": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mlk_re_layout_c": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "mlk_fp8_weight_repack": (c_int, [c_void_p, c_void_p, c_int64, c_void_p]),
    "mlk_stream_read": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    "mlk_mfma_probe": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_void_p]),
    "mlk_gemv_layout_a": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float,
                                  c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mlk_gemm_layout_a": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                  c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_size_t,
                                  c_void_p]),
    "mlk_gemm_layout_a_noalloc": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "mlk_gemm_noalloc_scratch_bytes": (c_size_t, []),
    "mlk_gemm_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int]),
    "mlk_gemm_counter_bytes": (c_size_t, []),
    "mlk_fused_routing_gate": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                       c_void_p, c_void_p, c_void_p]),
    "mlk_moe_align_tokens": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_void_p]),
    "mlk_fused_experts_compute": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int,
                                          c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_size_t, c_void_p]),
    "mlk_fused_moe": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                              c_int, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "mlk_moe_workspace_bytes": (c_size_t, [c_int, c_int, c_int, c_int, c_int]),
    "mlk_moe_plan": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
}

_lock = threading.Lock()
_lib = None


def load():
    """Load libmlk.so (once) and attach the prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "HIP extension not built: %s is missing. Run `python -m muxi_native_layout_kernels_amd.build` "
                "(needs hipcc); there is no CPU fallback." % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(code, what):
    """Turn a negative return code into a RuntimeError carrying the library's message."""
    if code != 0:
        msg = load().mlk_last_error()
        raise RuntimeError("%s failed (%d): %s" % (what, code, msg.decode() if msg else "?"))
