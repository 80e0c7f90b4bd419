"""ctypes binding of libmslk_amd.so (the C ABI declared in include/mslk_amd.h).

There is no fallback: if the shared library has not been built, `lib()` raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p, POINTER

_HERE = os.path.dirname(os.path.abspath(__file__))
# MSLK_AMD_LIBRARY overrides the location of the built library (e.g. an out-of-tree build).
LIB_PATH = os.environ.get("MSLK_AMD_LIBRARY") or os.path.join(_HERE, "libmslk_amd.so")

_lib = None

# name -> (restype, argtypes); mirrors include/mslk_amd.h one to one
SIGNATURES = {
    "mslk_amd_version": (c_char_p, []),
    "mslk_amd_last_error": (c_char_p, []),
    "mslk_amd_quantize_fp8_row": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                          c_void_p, c_void_p, c_void_p]),
    "mslk_amd_quantize_fp8_row_jagged": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                                 c_void_p, c_void_p, c_void_p, c_int, c_int64, c_void_p]),
    "mslk_amd_quantize_fp8_row_triton_arithmetic": (c_int, [c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                                            c_void_p, c_void_p, c_float, c_void_p, c_int, c_int64, c_void_p]),
    "mslk_amd_silu_mul_quant": (c_int, [c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64, c_void_p, c_void_p,
                                        c_void_p, c_void_p, c_int, c_void_p]),
    "mslk_amd_gather_scale_quant_dense_tokens": (c_int, [c_void_p, c_int, c_int64, c_int64, c_void_p, c_int, c_void_p, c_int,
                                                         c_int64, c_void_p, c_int, c_int64, c_int64, c_int64, c_void_p,
                                                         c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
    "mslk_amd_dequantize_fp8_row": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_void_p, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                          c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_static_scratch": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                                         c_int64, c_int64, c_int64, c_void_p]),
    "mslk_amd_static_scratch_bytes": (c_size_t, []),
    "mslk_amd_quantize_f8f8bf16_rowwise": (c_int, [c_void_p, c_int, c_int64, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                                   c_int64, c_int64, c_int64, c_void_p, c_void_p, c_void_p]),
    "mslk_amd_quantize_f8f8bf16_rowwise_supported": (c_int, [c_int64, c_int64, c_int64]),
    "mslk_amd_f8f8f16_rowwise": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p,
                                         c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "mslk_amd_f8f8_rowwise_preshuffle": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                                 c_int64, c_int64, c_int64, c_void_p]),
    "mslk_amd_f8f8_rowwise_preshuffle_workspace": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int,
                                                           c_int64, c_int64, c_int64, c_void_p, c_size_t, c_void_p]),
    "mslk_amd_preshuffle_b": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_workspace_bytes": (c_size_t, [c_int64, c_int64, c_int64]),
    "mslk_amd_f8f8bf16_rowwise_grouped": (c_int, [c_int, POINTER(c_void_p), POINTER(c_void_p), POINTER(c_void_p),
                                                  POINTER(c_void_p), POINTER(c_void_p), POINTER(c_int64),
                                                  POINTER(c_int64), POINTER(c_int64), c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_grouped_stacked": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                          c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_grouped_mm": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                                     c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_grouped_dynamic": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                                          c_int64, c_int64, c_int64, c_void_p, c_int, c_void_p]),
    "mslk_amd_f8f8bf16_rowwise_batched": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int64,
                                                  c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "mslk_amd_debug_cast_e4m3fn": (c_int, [c_void_p, c_int64, c_void_p, c_void_p]),
    "mslk_amd_debug_dispatch_name": (c_char_p, [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_int]),
    "mslk_amd_debug_stream_read": (c_int, [c_void_p, c_int64, c_int, c_int, c_void_p, c_void_p]),
    "mslk_amd_debug_mfma_loop": (c_int, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p]),
    "mslk_amd_debug_tile_streams": (c_int, [c_void_p, c_int64, c_void_p, c_int64, c_int64, c_int, c_int, c_int, c_void_p]),
    "mslk_amd_debug_gemm_phases": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int64, c_void_p, c_void_p]),
}


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"mslk_amd: {LIB_PATH} is missing. Build it with `python -m mslk_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no CPU or PyTorch fallback.")
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


def check(rc: int) -> None:
    """Turn a non-zero return code into the RuntimeError a TORCH_CHECK would have raised."""
    if rc != 0:
        raise RuntimeError(lib().mslk_amd_last_error().decode())
