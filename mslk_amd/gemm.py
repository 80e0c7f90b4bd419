"""`torch.ops.mslk.*` rowwise FP8 GEMM operators backed by the gfx950 HIP kernels.

The schema strings are the reference's (csrc/gemm/gemm_ops.cpp:31-44,88-96), so callers written
against `torch.ops.mslk.f8f8bf16_rowwise` etc. run unchanged.  When the reference's own library has
already defined a schema, only the GPU ("CUDA" dispatch key) kernel is replaced -- the same seam
the reference's Python kernels use (mslk/gemm/flydsl/preshuffle_gemm.py:433-475).

Validation and error messages follow the reference's ROCm host wrappers
(csrc/gemm/ck/fp8_rowwise/fp8fp8bf16_rowwise_gemm.hip:499-550,
 csrc/gemm/ck/fp8_rowwise_grouped/fp8_rowwise_grouped_gemm.hip:481-559,607-655), except that `bias`
is implemented (semantics of csrc/gemm/cutlass/f8f8bf16_rowwise/f8f8bf16_rowwise_common.cuh:150-198:
per-column fp32 or bf16 bias added after both scales) instead of rejected.
Only GPU kernels are registered: calling these ops with CPU tensors is a dispatcher error.
"""
from __future__ import annotations

import ctypes
from typing import List, Optional, Sequence

import torch

from . import _lib

FP8_DTYPE = torch.float8_e4m3fn

_SCHEMAS = {
    "f8f8bf16_rowwise": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? bias=None, bool use_fast_accum=True) -> Tensor",
    "f8f8bf16_rowwise_out": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor(a!) output, Tensor? bias=None, bool use_fast_accum=True) -> ()",
    "f8f8f16_rowwise": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? bias=None, bool use_fast_accum=True) -> Tensor",
    "f8f8bf16_rowwise_preshuffle": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? bias=None, bool use_fast_accum=True) -> Tensor",
    "f8f8f16_rowwise_preshuffle": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? bias=None, bool use_fast_accum=True) -> Tensor",
    "f8f8bf16_rowwise_grouped": "(Tensor[] XQ, Tensor[] WQ, Tensor[] x_scale, Tensor[] w_scale) -> Tensor[]",
    "f8f8bf16_rowwise_grouped_cat": "(Tensor[] XQ, Tensor[] WQ, Tensor[] x_scale, Tensor[] w_scale) -> Tensor",
    "f8f8bf16_rowwise_grouped_stacked": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor M_sizes) -> Tensor",
    "f8f8bf16_rowwise_grouped_dynamic": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor zero_start_index_M, bool zeroing_output_tensor=True) -> Tensor",
    "f8f8bf16_rowwise_grouped_mm": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? offsets, Tensor(a!) output) -> Tensor",
    "f8f8bf16_rowwise_batched": "(Tensor XQ, Tensor WQ, Tensor x_scale, Tensor w_scale, Tensor? bias=None, bool use_fast_accum=True, Tensor(a!)? output=None) -> Tensor",
    # no counterpart in the reference: its quantize_fp8_row -> f8f8bf16_rowwise pair as one operator (one launch at decode sizes)
    "quantize_f8f8bf16_rowwise": "(Tensor X, Tensor WQ, Tensor w_scale, Tensor? bias=None) -> (Tensor, Tensor, Tensor)",
}

_library = torch.library.Library("mslk", "FRAGMENT")


try:   # the raw handle of the current stream without building a Stream object (4 us -> 0.3 us per call)
    from torch._C import _cuda_getCurrentRawStream as _raw_stream
except ImportError:   # pragma: no cover
    _raw_stream = None


def _stream_ptr(device: torch.device) -> int:
    if _raw_stream is not None:
        return _raw_stream(device.index if device.index is not None else torch.cuda.current_device())
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """`with torch.cuda.device(d)` only when d is not already current (the switch costs microseconds)."""

    __slots__ = ("ctx",)

    def __init__(self, device: torch.device):
        self.ctx = None if device.index in (None, torch.cuda.current_device()) else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)


def _check(cond: bool, msg: str = "") -> None:
    if not cond:
        raise RuntimeError(msg or "Expected condition to be true (mslk_amd argument check)")


def _bias_args(bias: Optional[torch.Tensor], N: int, device: torch.device):
    if bias is None:
        return None, 0, None
    _check(bias.device == device, "bias must be on the same device as XQ")
    _check(bias.dtype in (torch.float32, torch.bfloat16), "Bias type must be bfloat16 or float32 if provided.")
    _check(bias.numel() == N, f"bias must have N={N} elements, got {bias.numel()}")
    b = bias.contiguous()
    return b.data_ptr(), (1 if b.dtype == torch.float32 else 2), b


def _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum, output=None, out_dtype=torch.bfloat16,
                  preshuffled=False):
    _check(XQ.dtype == WQ.dtype, f"XQ and WQ dtypes must match, got {XQ.dtype} vs {WQ.dtype}")
    _check(XQ.dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950, got {XQ.dtype}")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, "Scales must be float32.")
    _check(use_fast_accum, "AMD does not support disabling use_fast_accum.")
    _check(XQ.is_cuda and XQ.is_contiguous(), "XQ must be a contiguous GPU tensor")
    _check(WQ.is_cuda and WQ.is_contiguous(), "WQ must be a contiguous GPU tensor")
    _check(XQ.dim() >= 1 and WQ.dim() == 2, "XQ must be at least 1-D and WQ 2-D")
    N, K = WQ.shape
    _check(XQ.shape[-1] == K, f"XQ and WQ must share K, got {XQ.shape[-1]} vs {K}")
    M = 1
    for d in XQ.shape[:-1]:
        M *= d
    _check(x_scale.numel() == M, f"x_scale must have M={M} elements, got {x_scale.numel()}")
    _check(w_scale.numel() == N, f"w_scale must have N={N} elements, got {w_scale.numel()}")
    _check(x_scale.device == XQ.device and w_scale.device == XQ.device and WQ.device == XQ.device,
           "all operands must be on the same device")
    out_sizes = tuple(XQ.shape[:-1]) + (N,)
    if M == 0 or N == 0 or K == 0:
        # empty problem: zeros of the output shape (fp8fp8bf16_rowwise_gemm.hip:531-534)
        if output is not None:
            return output
        return torch.zeros(out_sizes, dtype=out_dtype, device=XQ.device)
    if output is not None:
        Y = output
        y_m = 1
        for d in Y.shape[:-1]:
            y_m *= d
        _check(y_m == M and Y.shape[-1] == N, "output has the wrong shape")
        _check(Y.dtype == out_dtype, f"output must be {out_dtype}")
        _check(Y.is_cuda and Y.is_contiguous() and Y.device == XQ.device, "output must be a contiguous GPU tensor")
    else:
        Y = torch.empty(out_sizes, dtype=out_dtype, device=XQ.device)
    xs = x_scale.contiguous()
    ws = w_scale.contiguous()
    bias_ptr, bias_code, _keep = _bias_args(bias, N, XQ.device)
    if preshuffled:
        _check(N % 16 == 0 and K % 64 == 0, f"pre-shuffled weights need N % 16 == 0 and K % 64 == 0, got N={N} K={K}")
        # few output tiles and a long K: room for the fp32 sums of the K slices, as for row-major weights below
        wsp_ptr, wsp_bytes = None, _lib.lib().mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
        if wsp_bytes:
            wsp = torch.empty(wsp_bytes, dtype=torch.uint8, device=XQ.device)
            wsp_ptr = wsp.data_ptr()
        with _on_device(XQ.device):
            _lib.check(_lib.lib().mslk_amd_f8f8_rowwise_preshuffle_workspace(
                XQ.data_ptr(), WQ.data_ptr(), xs.data_ptr(), ws.data_ptr(), bias_ptr, bias_code, Y.data_ptr(),
                1 if out_dtype == torch.float16 else 0, M, N, K, wsp_ptr, wsp_bytes, _stream_ptr(XQ.device)))
        return Y
    wsp_ptr, wsp_bytes = None, 0
    if K % 16 or XQ.data_ptr() % 16 or WQ.data_ptr() % 16:
        # rows the 16-byte loads cannot fetch: room for copies with K rounded up (the caching allocator's block, so the
        # call stays capturable); the library pads into it and runs the MFMA kernels on the copies
        wsp_bytes = (M + N) * ((K + 15) // 16 * 16)
        wsp = torch.empty(wsp_bytes, dtype=torch.uint8, device=XQ.device)
        wsp_ptr = wsp.data_ptr()
    else:
        # few output tiles and a long K: the library splits K when it is given room for the fp32 sums of the slices
        wsp_bytes = _lib.lib().mslk_amd_f8f8bf16_rowwise_workspace_bytes(M, N, K)
        if wsp_bytes:
            wsp = torch.empty(wsp_bytes, dtype=torch.uint8, device=XQ.device)
            wsp_ptr = wsp.data_ptr()
    with _on_device(XQ.device):
        fn = _lib.lib().mslk_amd_f8f8f16_rowwise if out_dtype == torch.float16 else _lib.lib().mslk_amd_f8f8bf16_rowwise
        _lib.check(fn(XQ.data_ptr(), WQ.data_ptr(), xs.data_ptr(), ws.data_ptr(), bias_ptr, bias_code, Y.data_ptr(),
                      M, N, K, wsp_ptr, wsp_bytes, _stream_ptr(XQ.device)))
    return Y


def f8f8bf16_rowwise(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    return _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum)


def f8f8bf16_rowwise_out(XQ, WQ, x_scale, w_scale, output, bias=None, use_fast_accum=True):
    _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum, output)


def quantize_f8f8bf16_rowwise(X, WQ, w_scale, bias=None):
    """bf16 activations in, bf16 out: `quantize_fp8_row(X, use_triton=False)` followed by `f8f8bf16_rowwise`, returning
    (Y, XQ, x_scale) -- the pair every decode step of a caller of the reference issues (bench/gemm/gemm_ops.py:593-673).
    For 1 <= M <= 4 rows of bf16 with K % 128 == 0 (K >= 1024) it is ONE launch (every workgroup quantizes the rows itself; XQ and
    x_scale are the bits the stand-alone quantizer returns); other shapes run the two kernels."""
    _check(WQ.dtype == FP8_DTYPE, f"WQ must be {FP8_DTYPE} on gfx950, got {WQ.dtype}")
    _check(w_scale.dtype == torch.float32, "Scales must be float32.")
    _check(X.is_cuda and WQ.is_cuda and WQ.is_contiguous() and WQ.dim() == 2, "WQ must be a contiguous 2-D GPU tensor")
    _check(X.dim() >= 1 and X.shape[-1] == WQ.shape[1], f"X and WQ must share K, got {X.shape[-1]} vs {WQ.shape[1]}")
    N, K = WQ.shape
    M = 1
    for d in X.shape[:-1]:
        M *= d
    _check(w_scale.numel() == N, f"w_scale must have N={N} elements, got {w_scale.numel()}")
    _check(w_scale.device == X.device and WQ.device == X.device, "all operands must be on the same device")
    L = _lib.lib()
    x2 = X.reshape(M, K) if M else X
    one_launch = (X.dtype == torch.bfloat16 and M > 0 and L.mslk_amd_quantize_f8f8bf16_rowwise_supported(M, N, K)
                  and x2.stride(-1) == 1 and x2.stride(0) % 8 == 0 and x2.data_ptr() % 16 == 0 and WQ.data_ptr() % 16 == 0)
    if not one_launch:
        from .quantize import quantize_fp8_row
        XQ, x_scale = quantize_fp8_row(X, use_triton=False)
        return _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, True), XQ, x_scale
    ws = w_scale.contiguous()
    bias_ptr, bias_code, _keep = _bias_args(bias, N, X.device)
    Y = torch.empty(tuple(X.shape[:-1]) + (N,), dtype=torch.bfloat16, device=X.device)
    XQ = torch.empty(X.shape, dtype=FP8_DTYPE, device=X.device)
    x_scale = torch.empty(X.shape[:-1], dtype=torch.float32, device=X.device)
    with _on_device(X.device):
        _lib.check(L.mslk_amd_quantize_f8f8bf16_rowwise(
            x2.data_ptr(), 0, x2.stride(0), WQ.data_ptr(), ws.data_ptr(), bias_ptr, bias_code, Y.data_ptr(), M, N, K,
            XQ.data_ptr(), x_scale.data_ptr(), _stream_ptr(X.device)))
    return Y, XQ, x_scale


def f8f8f16_rowwise(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    """Same GEMM with an fp16 result (fp8fp8fp16_rowwise_gemm.hip:66-133)."""
    return _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum, None, torch.float16)


def f8f8bf16_rowwise_preshuffle(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    """f8f8bf16_rowwise on weights pre-shuffled by `ck_preshuffle(wq, 16)` / `preshuffle_b_mfma(wq)`
    (fp8_rowwise_preshuffle_gemm.hip:93-171)."""
    return _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum, None, torch.bfloat16, True)


def f8f8f16_rowwise_preshuffle(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    """fp16-output variant.  (The reference registers its bf16 function under this name too,
    gemm_ops.cpp:145; the schema and the fp16 wrapper at fp8_rowwise_preshuffle_gemm.hip:160-171 say fp16.)"""
    return _rowwise_impl(XQ, WQ, x_scale, w_scale, bias, use_fast_accum, None, torch.float16, True)


def preshuffle_b_mfma(src: torch.Tensor) -> torch.Tensor:
    """FP8 weights [N, K] or [G, N, K] -> the blocked order [N/16][K/64][4][16][16 B] the *_preshuffle GEMMs
    read (mslk/quantize/shuffle.py:208-246).  Same shape and dtype as `src`; out of place."""
    _check(src.is_cuda and src.is_contiguous(), "preshuffle_b_mfma: src must be a contiguous GPU tensor")
    _check(src.element_size() == 1 and src.dim() in (2, 3), "preshuffle_b_mfma: src must be an 8-bit [N, K] or [G, N, K] tensor")
    N, K = src.shape[-2], src.shape[-1]
    if N % 16 or K % 64:
        raise ValueError(f"preshuffle_b_mfma needs N % 16 == 0 and K % 64 == 0, got N={N} K={K}")
    G = src.shape[0] if src.dim() == 3 else 1
    dst = torch.empty_like(src)
    if src.numel():
        with _on_device(src.device):
            _lib.check(_lib.lib().mslk_amd_preshuffle_b(src.data_ptr(), dst.data_ptr(), G, N, K, _stream_ptr(src.device)))
    return dst


def ck_preshuffle(src: torch.Tensor, NXdl: int = 16) -> torch.Tensor:
    """Reference name for the same re-layout of one [N, K] matrix (mslk/quantize/shuffle.py:182-205);
    only the 16-row wave tile the GEMM reads is supported."""
    _check(NXdl == 16, "ck_preshuffle: only NXdl = 16 is supported")
    _check(src.dim() == 2, "ck_preshuffle: src must be [N, K]")
    return preshuffle_b_mfma(src)


def _check_grouped(XQ: Sequence[torch.Tensor], WQ, x_scale, w_scale):
    """Argument checks of the TensorList ops; one pass over the groups (this runs on every call of a decode loop, so the
    common case costs a few comparisons per group and messages are only built on failure)."""
    G = len(XQ)
    _check(G == len(WQ) == len(x_scale) == len(w_scale), "All inputs must have the same number of groups.")
    if G == 0:
        return
    dev, f32 = XQ[0].device, torch.float32
    _check(XQ[0].dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950, got {XQ[0].dtype}")
    for x, w, xs, ws in zip(XQ, WQ, x_scale, w_scale):
        xsh, wsh = x.shape, w.shape
        if not (x.is_cuda and w.is_cuda and x.is_contiguous() and w.is_contiguous()):
            _check(x.is_cuda and x.is_contiguous(), "XQ tensors must be contiguous GPU tensors")
            _check(False, "WQ tensors must be contiguous GPU tensors")
        _check(len(xsh) == 2 and len(wsh) == 2, "Inputs must be 2D.")
        if w.dtype != FP8_DTYPE or x.dtype != FP8_DTYPE:
            other = w.dtype if w.dtype != FP8_DTYPE else x.dtype
            _check(False, f"XQ and WQ dtypes must match, got {FP8_DTYPE} vs {other}")
        _check(wsh[0] >= 512 and wsh[1] >= 512,
               "N and K must be at least 512 for grouped gemm. For smaller inputs, consider unrolling.")
        _check(xs.dtype == f32 and ws.dtype == f32, "Scales must be float32.")
        _check(xsh[1] == wsh[1], "XQ and WQ of a group must share K")
        _check(xs.numel() == xsh[0] and ws.numel() == wsh[0], "scale sizes must match M and N of their group")
        _check(x.device == dev and w.device == dev and xs.device == dev and ws.device == dev,
               "all operands must be on the same device")


def _launch_grouped(XQ, WQ, x_scale, w_scale, outs: List[torch.Tensor]) -> None:
    G = len(XQ)
    xs = [s if s.is_contiguous() else s.contiguous() for s in x_scale]
    ws = [s if s.is_contiguous() else s.contiguous() for s in w_scale]
    PtrArr = ctypes.c_void_p * G
    I64Arr = ctypes.c_int64 * G
    dev = XQ[0].device
    with _on_device(dev):
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped(
            G, PtrArr(*[t.data_ptr() for t in XQ]), PtrArr(*[t.data_ptr() for t in WQ]),
            PtrArr(*[t.data_ptr() for t in xs]), PtrArr(*[t.data_ptr() for t in ws]),
            PtrArr(*[t.data_ptr() for t in outs]),
            I64Arr(*[t.shape[0] for t in XQ]), I64Arr(*[t.shape[0] for t in WQ]), I64Arr(*[t.shape[1] for t in WQ]),
            _stream_ptr(dev)))


def f8f8bf16_rowwise_grouped(XQ, WQ, x_scale, w_scale) -> List[torch.Tensor]:
    """TensorList grouped GEMM; the outputs are views into ONE flat bf16 buffer
    (fp8_rowwise_grouped_gemm.hip:528-529,553-557)."""
    _check_grouped(XQ, WQ, x_scale, w_scale)
    if len(XQ) == 0:
        return []
    Ms = [x.shape[0] for x in XQ]
    Ns = [w.shape[0] for w in WQ]
    if Ns.count(Ns[0]) == len(Ns):   # one N: the row blocks of a [sum M, N] buffer are the same views, made by one call
        outs = list(torch.empty((sum(Ms), Ns[0]), dtype=torch.bfloat16, device=XQ[0].device).split(Ms))
    else:
        sizes = [m * n for m, n in zip(Ms, Ns)]
        flat = torch.empty(sum(sizes), dtype=torch.bfloat16, device=XQ[0].device)
        outs = [t.view(m, n) for t, m, n in zip(flat.split(sizes), Ms, Ns)]
    _launch_grouped(XQ, WQ, x_scale, w_scale, outs)
    return outs


def f8f8bf16_rowwise_grouped_cat(XQ, WQ, x_scale, w_scale) -> torch.Tensor:
    """Same computation, outputs concatenated along M (all groups must share N)."""
    _check_grouped(XQ, WQ, x_scale, w_scale)
    _check(len(XQ) > 0, "at least one group is required")
    N = WQ[0].shape[0]
    _check(all(w.shape[0] == N for w in WQ), "all groups must share N to concatenate outputs")
    total_M = sum(x.shape[0] for x in XQ)
    Y = torch.empty((total_M, N), dtype=torch.bfloat16, device=XQ[0].device)
    outs = list(Y.split([x.shape[0] for x in XQ], dim=0))
    _launch_grouped(XQ, WQ, x_scale, w_scale, outs)
    return Y


def f8f8bf16_rowwise_grouped_stacked(XQ, WQ, x_scale, w_scale, M_sizes) -> torch.Tensor:
    """XQ [total_M, K], WQ [G, N, K], x_scale [total_M], w_scale [G, N], M_sizes int64 [G] on the GPU
    (fp8_rowwise_grouped_gemm.hip:607-655).  M_sizes is never read on the host."""
    _check(XQ.is_cuda and XQ.is_contiguous() and WQ.is_cuda and WQ.is_contiguous(), "XQ/WQ must be contiguous GPU tensors")
    _check(XQ.dim() == 2 and WQ.dim() == 3, "XQ must be 2-D [total_M, K] and WQ 3-D [G, N, K]")
    _check(XQ.dtype == WQ.dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, "Scales must be float32.")
    _check(M_sizes.is_cuda and M_sizes.dtype == torch.int64, "M_sizes must be an int64 GPU tensor")
    total_M, K = XQ.shape
    G, N, Kw = WQ.shape
    _check(K == Kw, "XQ and WQ must share K")
    _check(M_sizes.numel() == G, "M_sizes must have one entry per group")
    _check(x_scale.numel() == total_M and w_scale.numel() == G * N, "scale sizes must match total_M and G*N")
    Y = torch.empty((total_M, N), dtype=torch.bfloat16, device=XQ.device)
    if total_M == 0 or N == 0 or G == 0:
        return Y
    if K == 0:
        return Y.zero_()
    xs, ws, ms = x_scale.contiguous(), w_scale.contiguous(), M_sizes.contiguous()
    with _on_device(XQ.device):
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped_stacked(
            XQ.data_ptr(), WQ.data_ptr(), xs.data_ptr(), ws.data_ptr(), ms.data_ptr(), G, total_M, N, K,
            Y.data_ptr(), _stream_ptr(XQ.device)))
    return Y


# group layout codes of mslk_amd_f8f8bf16_rowwise_grouped_mm (include/mslk_amd.h)
_GROUPS_M_OFFSETS, _GROUPS_N_OFFSETS, _GROUPS_K_OFFSETS, _GROUPS_UNIFORM = 1, 2, 3, 4


def f8f8bf16_rowwise_grouped_mm(XQ, WQ, x_scale, w_scale, offsets, output) -> torch.Tensor:
    """Grouped GEMM in the torch._grouped_mm convention (fp8_rowwise_grouped_gemm.hip:720-845): the
    ranks of XQ / WQ select which dimension varies per group, `offsets` (int32, on the GPU, never
    read on the host) holds the cumulative group ends along it, and the result is written into
    `output`, which is returned.

      XQ [total_M, K], WQ [G, N, K]   offsets over M   output [total_M, N]
      XQ [G, M, K],    WQ [total_N, K] offsets over N   output [M, total_N]
      XQ [G, M, K],    WQ [G, N, K]    no offsets       output [G, M, N]
      XQ [M, total_K], WQ [N, total_K] offsets over K   output [G, M, N]
    """
    _check(XQ.is_cuda and XQ.is_contiguous() and WQ.is_cuda and WQ.is_contiguous(), "XQ/WQ must be contiguous GPU tensors")
    _check(XQ.dtype == WQ.dtype, f"XQ and WQ dtypes must match, got {XQ.dtype} vs {WQ.dtype}")
    _check(XQ.dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950, got {XQ.dtype}")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, "Scales must be float32.")
    _check(x_scale.is_contiguous() and w_scale.is_contiguous(), "scales must be contiguous")

    def need_offsets(what):
        _check(offsets is not None, f"Must pass offsets for 2D input {what}.")
        _check(offsets.dtype == torch.int32, "offsets must be int32.")
        _check(offsets.is_cuda and offsets.is_contiguous() and offsets.dim() == 1, "offsets must be a 1-D contiguous GPU tensor")
        return offsets.shape[0]

    if XQ.dim() == 2 and WQ.dim() == 3:
        G = need_offsets("XQ")
        M, N, K = XQ.shape[0], WQ.shape[1], WQ.shape[2]
        layout = _GROUPS_M_OFFSETS
        _check(XQ.shape[1] == K and WQ.shape[0] == G, "XQ shape must be (total_M, K) and WQ shape must be (G, N, K).")
        _check(x_scale.shape[0] == M, "x_scale shape must be (total_M).")
        _check(w_scale.dim() == 2 and w_scale.shape[0] == G and w_scale.shape[1] == N, "w_scale shape must be (G, N).")
        _check(output.dim() == 2 and output.shape[0] == M and output.shape[1] == N, "out shape must be (total_M, N).")
    elif XQ.dim() == 3 and WQ.dim() == 2:
        G = need_offsets("WQ")
        M, N, K = XQ.shape[1], WQ.shape[0], WQ.shape[1]
        layout = _GROUPS_N_OFFSETS
        _check(XQ.shape[0] == G and XQ.shape[2] == K, "XQ shape must be (G, M, K) and WQ shape must be (total_N, K).")
        _check(x_scale.dim() == 2 and x_scale.shape[0] == G and x_scale.shape[1] == M, "x_scale shape must be (G, M).")
        _check(w_scale.shape[0] == N, "w_scale shape must be (total_N).")
        _check(output.dim() == 2 and output.shape[0] == M and output.shape[1] == N, "out shape must be (M, total_N).")
    elif XQ.dim() == 3 and WQ.dim() == 3:
        _check(offsets is None, "Offsets should not be passed for 3D-3D inputs.")
        G, M, K = XQ.shape
        N = WQ.shape[1]
        layout = _GROUPS_UNIFORM
        _check(WQ.shape[0] == G and WQ.shape[2] == K, "XQ shape must be (G, M, K) and WQ shape must be (G, N, K).")
        _check(x_scale.dim() == 2 and x_scale.shape[0] == G and x_scale.shape[1] == M, "x_scale shape must be (G, M).")
        _check(w_scale.dim() == 2 and w_scale.shape[0] == G and w_scale.shape[1] == N, "w_scale shape must be (G, N).")
        _check(output.dim() == 3 and tuple(output.shape) == (G, M, N), "out shape must be (G, M, N).")
    elif XQ.dim() == 2 and WQ.dim() == 2:
        G = need_offsets("s XQ and WQ")
        M, N, K = XQ.shape[0], WQ.shape[0], XQ.shape[1]
        layout = _GROUPS_K_OFFSETS
        _check(WQ.shape[1] == K, "XQ shape must be (M, total_K) and WQ shape must be (N, total_K).")
        _check(x_scale.shape[0] == G * M, "x_scale shape must be (G * M).")
        _check(w_scale.shape[0] == G * N, "w_scale shape must be (G * N).")
        _check(output.dim() == 3 and tuple(output.shape) == (G, M, N), "out shape must be (G, M, N).")
    else:
        _check(False, "Invalid input shapes. Must be one of 2D-2D, 3D-3D, 2D-3D, 3D-2D.")
    if layout != _GROUPS_N_OFFSETS:
        _check(N % 8 == 0, "N must be divisible by 8.")
    _check(output.dtype == torch.bfloat16 and output.is_cuda and output.is_contiguous() and output.device == XQ.device,
           "output must be a contiguous bfloat16 GPU tensor on the device of XQ")
    _check(WQ.device == XQ.device and x_scale.device == XQ.device and w_scale.device == XQ.device and
           (offsets is None or offsets.device == XQ.device), "all operands must be on the same device")
    if output.numel() == 0:
        return output
    with _on_device(XQ.device):
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped_mm(
            XQ.data_ptr(), WQ.data_ptr(), x_scale.data_ptr(), w_scale.data_ptr(),
            None if offsets is None else offsets.data_ptr(), layout, G, M, N, K, output.data_ptr(),
            _stream_ptr(XQ.device)))
    return output


def f8f8bf16_rowwise_grouped_dynamic(XQ, WQ, x_scale, w_scale, zero_start_index_M, zeroing_output_tensor=True) -> torch.Tensor:
    """XQ [G, M, K], WQ [G, N, K] -> bf16 [G, M, N]; only the first zero_start_index_M[g] rows of group
    g are computed, the others are zero (or uninitialised when zeroing_output_tensor is False).
    Deprecated in the reference (fp8_rowwise_grouped_gemm.hip:656-714) but still registered."""
    _check(XQ.dim() == 3, "Input XQ must be 3D (G,M,K).")
    _check(WQ.dim() == 3, "Input WQ must be 3D (G,N,K).")
    _check(XQ.is_cuda and XQ.is_contiguous() and WQ.is_cuda and WQ.is_contiguous(), "XQ/WQ must be contiguous GPU tensors")
    _check(XQ.dtype == WQ.dtype, f"XQ and WQ dtypes must match, got {XQ.dtype} vs {WQ.dtype}")
    _check(XQ.dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950, got {XQ.dtype}")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, "Scales must be float32.")
    G, M, K = XQ.shape
    N = WQ.shape[1]
    _check(WQ.shape[0] == G and x_scale.numel() == G * M and w_scale.numel() == G * N and WQ.shape[2] == K,
           "All inputs must have the same number of groups.")
    _check(N >= 512 and K >= 512, "N and K must be at least 512 for grouped gemm. For smaller inputs, consider unrolling.")
    zs = zero_start_index_M
    _check(zs.is_cuda and zs.dtype == torch.int64 and zs.numel() == G, "zero_start_index_M must be an int64 GPU tensor with G entries")
    _check(WQ.device == XQ.device and x_scale.device == XQ.device and w_scale.device == XQ.device and zs.device == XQ.device,
           "all operands must be on the same device")
    Y = torch.empty((G, M, N), dtype=torch.bfloat16, device=XQ.device)
    if Y.numel() == 0:
        return Y
    xs, ws, zs = x_scale.contiguous(), w_scale.contiguous(), zs.contiguous()
    with _on_device(XQ.device):
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_grouped_dynamic(
            XQ.data_ptr(), WQ.data_ptr(), xs.data_ptr(), ws.data_ptr(), zs.data_ptr(), G, M, N, K, Y.data_ptr(),
            1 if zeroing_output_tensor else 0, _stream_ptr(XQ.device)))
    return Y


def f8f8bf16_rowwise_batched(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True, output=None) -> torch.Tensor:
    """XQ [B, M, K], WQ [B, N, K], x_scale [B, M], w_scale [B, N] -> bf16 [B, M, N]
    (fp8_rowwise_batched_gemm.hip:199-254).  `bias` [B, N] (fp32 or bf16) is added per batch as the
    reference's CUTLASS build does (f8f8bf16_rowwise_batched_common.cuh:272-275); its ROCm build
    accepts the argument and drops it."""
    _check(XQ.dim() == 3 and WQ.dim() == 3, "Inputs must have 3 dimensions, with the first being batch.")
    _check(XQ.dtype == WQ.dtype, f"XQ and WQ dtypes must match, got {XQ.dtype} vs {WQ.dtype}")
    _check(XQ.dtype == FP8_DTYPE, f"XQ and WQ must be {FP8_DTYPE} on gfx950, got {XQ.dtype}")
    _check(x_scale.dtype == torch.float32 and w_scale.dtype == torch.float32, "Scales must be float32.")
    _check(use_fast_accum, "AMD does not support disabling use_fast_accum.")
    _check(XQ.is_cuda and XQ.is_contiguous(), "XQ must be a contiguous GPU tensor")
    _check(WQ.is_cuda and WQ.is_contiguous(), "WQ must be a contiguous GPU tensor")
    B, M, K = XQ.shape
    N = WQ.shape[1]
    _check(WQ.shape[0] == B and WQ.shape[2] == K, "XQ must be (B, M, K) and WQ (B, N, K)")
    _check(x_scale.numel() == B * M and w_scale.numel() == B * N, "scale sizes must match B*M and B*N")
    _check(WQ.device == XQ.device and x_scale.device == XQ.device and w_scale.device == XQ.device,
           "all operands must be on the same device")
    if output is not None:
        Y = output
        _check(Y.dim() == 3, "Output tensor must have three dimensions.")
        _check(tuple(Y.shape) == (B, M, N), "output has the wrong shape")
        _check(Y.dtype == torch.bfloat16, "output must be bfloat16")
        _check(Y.is_cuda and Y.is_contiguous() and Y.device == XQ.device, "output must be a contiguous GPU tensor")
    else:
        Y = torch.empty((B, M, N), dtype=torch.bfloat16, device=XQ.device)
    if Y.numel() == 0:
        return Y
    xs, ws = x_scale.contiguous(), w_scale.contiguous()
    bias_ptr, bias_code, _keep = _bias_args(bias, B * N, XQ.device)
    with _on_device(XQ.device):
        _lib.check(_lib.lib().mslk_amd_f8f8bf16_rowwise_batched(
            XQ.data_ptr(), WQ.data_ptr(), xs.data_ptr(), ws.data_ptr(), bias_ptr, bias_code, B, M, N, K,
            Y.data_ptr(), _stream_ptr(XQ.device)))
    return Y


# ---------------------------------------------------------------------------------------------
# registration
# ---------------------------------------------------------------------------------------------
_IMPLS = {
    "f8f8bf16_rowwise": f8f8bf16_rowwise,
    "f8f8bf16_rowwise_out": f8f8bf16_rowwise_out,
    "f8f8f16_rowwise": f8f8f16_rowwise,
    "f8f8bf16_rowwise_preshuffle": f8f8bf16_rowwise_preshuffle,
    "f8f8f16_rowwise_preshuffle": f8f8f16_rowwise_preshuffle,
    "f8f8bf16_rowwise_grouped": f8f8bf16_rowwise_grouped,
    "f8f8bf16_rowwise_grouped_cat": f8f8bf16_rowwise_grouped_cat,
    "f8f8bf16_rowwise_grouped_stacked": f8f8bf16_rowwise_grouped_stacked,
    "f8f8bf16_rowwise_grouped_dynamic": f8f8bf16_rowwise_grouped_dynamic,
    "f8f8bf16_rowwise_grouped_mm": f8f8bf16_rowwise_grouped_mm,
    "f8f8bf16_rowwise_batched": f8f8bf16_rowwise_batched,
    "quantize_f8f8bf16_rowwise": quantize_f8f8bf16_rowwise,
}


def _fake_quantize_rowwise(X, WQ, w_scale, bias=None):
    return (torch.empty(tuple(X.shape[:-1]) + (WQ.shape[0],), dtype=torch.bfloat16, device=X.device),
            torch.empty(X.shape, dtype=FP8_DTYPE, device=X.device),
            torch.empty(X.shape[:-1], dtype=torch.float32, device=X.device))


def _fake_rowwise(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    # mslk/gemm/_meta.py:26-50, generalised to any number of leading dims
    return torch.empty(tuple(XQ.shape[:-1]) + (WQ.shape[0],), dtype=torch.bfloat16, device=XQ.device)


def _fake_rowwise_f16(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True):
    # mslk/gemm/_meta.py:516-529, generalised to any number of leading dims
    return torch.empty(tuple(XQ.shape[:-1]) + (WQ.shape[0],), dtype=torch.float16, device=XQ.device)


def _fake_rowwise_out(XQ, WQ, x_scale, w_scale, output, bias=None, use_fast_accum=True):
    return None


def _fake_grouped(XQ, WQ, x_scale, w_scale):
    # as the kernel (and the reference): views into one flat buffer
    if len(XQ) == 0:
        return []
    sizes = [x.shape[0] * w.shape[0] for x, w in zip(XQ, WQ)]
    flat = torch.empty(sum(sizes), dtype=torch.bfloat16, device=XQ[0].device)
    return [t.view(x.shape[0], w.shape[0]) for t, x, w in zip(flat.split(sizes), XQ, WQ)]


def _fake_grouped_cat(XQ, WQ, x_scale, w_scale):
    return torch.empty((sum(x.shape[0] for x in XQ), WQ[0].shape[0]), dtype=torch.bfloat16, device=XQ[0].device)


def _fake_grouped_stacked(XQ, WQ, x_scale, w_scale, M_sizes):
    # mslk/gemm/_meta.py:114-126
    return torch.empty((XQ.shape[0], WQ.shape[1]), dtype=torch.bfloat16, device=XQ.device)


def _fake_grouped_dynamic(XQ, WQ, x_scale, w_scale, zero_start_index_M, zeroing_output_tensor=True):
    return torch.empty((XQ.shape[0], XQ.shape[1], WQ.shape[1]), dtype=torch.bfloat16, device=XQ.device)


def _fake_grouped_mm(XQ, WQ, x_scale, w_scale, offsets, output):
    return output


def _fake_batched(XQ, WQ, x_scale, w_scale, bias=None, use_fast_accum=True, output=None):
    # mslk/gemm/_meta.py:68-83
    if output is not None:
        return output
    return torch.empty((XQ.shape[0], XQ.shape[1], WQ.shape[1]), dtype=torch.bfloat16, device=XQ.device)


_FAKES = {
    "f8f8bf16_rowwise": _fake_rowwise,
    "f8f8bf16_rowwise_out": _fake_rowwise_out,
    "f8f8f16_rowwise": _fake_rowwise_f16,
    "f8f8bf16_rowwise_preshuffle": _fake_rowwise,
    "f8f8f16_rowwise_preshuffle": _fake_rowwise_f16,
    "f8f8bf16_rowwise_grouped": _fake_grouped,
    "f8f8bf16_rowwise_grouped_cat": _fake_grouped_cat,
    "f8f8bf16_rowwise_grouped_stacked": _fake_grouped_stacked,
    "f8f8bf16_rowwise_grouped_dynamic": _fake_grouped_dynamic,
    "f8f8bf16_rowwise_grouped_mm": _fake_grouped_mm,
    "f8f8bf16_rowwise_batched": _fake_batched,
    "quantize_f8f8bf16_rowwise": _fake_quantize_rowwise,
}


def _register() -> None:
    for name, schema in _SCHEMAS.items():
        already = hasattr(torch.ops.mslk, name)
        if not already:
            _library.define(name + schema)
        # GPU kernel: on ROCm builds of PyTorch HIP tensors dispatch on the "CUDA" key.
        _library.impl(name, _IMPLS[name], "CUDA", allow_override=True) if already else _library.impl(name, _IMPLS[name], "CUDA")
        if not already:
            torch.library.register_fake(f"mslk::{name}", _FAKES[name], lib=_library)


_register()
