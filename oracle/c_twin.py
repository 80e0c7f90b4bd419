"""ctypes loader for oracle/liboracle_fp8.so (the scalar C twin).  TEST INFRASTRUCTURE ONLY."""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "liboracle_fp8.so")
_lib = None
_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


def build() -> str:
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "liboracle_fp8.so"])
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        L = ctypes.CDLL(_SO)
        L.oracle_e4m3fn_from_f32.restype = ctypes.c_uint8
        L.oracle_e4m3fn_from_f32.argtypes = [ctypes.c_float]
        L.oracle_e4m3fn_to_f32.restype = ctypes.c_float
        L.oracle_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.oracle_e4m3fn_cast.restype = None
        L.oracle_e4m3fn_cast.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        L.oracle_quantize_rows.restype = None
        L.oracle_quantize_rows.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_int64,
                                           ctypes.c_int64, ctypes.c_int, ctypes.c_double,
                                           ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p]
        L.oracle_dequant_gemm.restype = None
        L.oracle_dequant_gemm.argtypes = [ctypes.c_void_p] * 5 + [ctypes.c_int64] * 3 + [ctypes.c_void_p]
        L.oracle_count_division_mismatches.restype = ctypes.c_uint64
        L.oracle_count_division_mismatches.argtypes = [ctypes.c_int, ctypes.c_uint32, ctypes.c_uint32,
                                                       ctypes.POINTER(ctypes.c_uint32), ctypes.POINTER(ctypes.c_uint32)]
        _lib = L
    return _lib


def count_division_mismatches(dtype: torch.dtype, first_c_bits: int = 0, end_c_bits: int = 0):
    """Pairs (row maximum c, element x) of 16-bit values, c bits in [first_c_bits, end_c_bits), whose e4m3 code differs
    between the IEEE division x / (c / 448) and the reciprocal + two fused multiply-adds the quantizer kernel uses.
    Returns (count, first offending pair, last offending pair) with pairs as (c bits << 16 | x bits)."""
    fb, lb = ctypes.c_uint32(0), ctypes.c_uint32(0)
    n = lib().oracle_count_division_mismatches(_DTYPE_CODE[dtype], first_c_bits, end_c_bits, ctypes.byref(fb), ctypes.byref(lb))
    return int(n), fb.value, lb.value


def e4m3fn_cast(x: torch.Tensor) -> torch.Tensor:
    """fp32 tensor -> uint8 e4m3fn codes via the C twin."""
    x = x.detach().cpu().contiguous().to(torch.float32)
    out = torch.empty(x.shape, dtype=torch.uint8)
    lib().oracle_e4m3fn_cast(x.data_ptr(), x.numel(), out.data_ptr())
    return out


def quantize_rows(a: torch.Tensor, scale_ub: float | None = None):
    """2-D contiguous bf16/fp16/fp32 CPU tensor -> (uint8 codes [R,K], fp32 scale [R])."""
    assert a.dim() == 2 and a.device.type == "cpu"
    a = a.contiguous()
    R, K = a.shape
    codes = torch.empty((R, K), dtype=torch.uint8)
    scale = torch.empty((R,), dtype=torch.float32)
    lib().oracle_quantize_rows(a.data_ptr(), _DTYPE_CODE[a.dtype], R, K, K,
                               0 if scale_ub is None else 1, 0.0 if scale_ub is None else float(scale_ub),
                               codes.data_ptr(), K, scale.data_ptr())
    return codes, scale


def dequant_gemm(xq_codes: torch.Tensor, wq_codes: torch.Tensor, xs: torch.Tensor, ws: torch.Tensor,
                 bias: torch.Tensor | None = None) -> torch.Tensor:
    """Brute-force float64 triple loop over uint8 e4m3fn codes."""
    xq_codes = xq_codes.contiguous(); wq_codes = wq_codes.contiguous()
    M, K = xq_codes.shape
    N = wq_codes.shape[0]
    xs = xs.contiguous().float(); ws = ws.contiguous().float()
    b = None if bias is None else bias.contiguous().float()
    y = torch.empty((M, N), dtype=torch.float64)
    lib().oracle_dequant_gemm(xq_codes.data_ptr(), wq_codes.data_ptr(), xs.data_ptr(), ws.data_ptr(),
                              None if b is None else b.data_ptr(), M, N, K, y.data_ptr())
    return y
