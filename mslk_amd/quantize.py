"""Row-wise FP8 quantization behind the reference's Python interface.

`quantize_fp8_row` keeps the signature, the operator name (`triton::quantize_fp8_row`) and the dispatch of the
reference function (mslk/quantize/triton/fp8_quantize.py:319-378): `use_triton=True` selects the arithmetic of its
GPU kernel, `use_triton=False` the bits of its torch emulation (356-378).  `quantize_fp8_per_row`
(`mslk::quantize_fp8_per_row`) always gives the latter.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

FP8_DTYPE = torch.float8_e4m3fn  # gfx950 is OCP FP8 (reference: mslk/utils/device.py:135-160)
_DTYPE_CODE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}


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


def _quantize_launch(a: torch.Tensor, scale_ub: Optional[torch.Tensor], zero_start_index_M: Optional[torch.Tensor],
                     align_rows_to: Optional[int], triton_eps: Optional[float]) -> Tuple[torch.Tensor, torch.Tensor]:
    """One quantizer launch.  `triton_eps` None: the arithmetic of the reference's torch branch; a float: the arithmetic of
    its Triton kernel with that lower bound of amax."""
    if a.dtype not in _DTYPE_CODE:
        raise RuntimeError(f"quantize_fp8_row: unsupported input dtype {a.dtype} (bf16, fp16, fp32 are supported)")
    if a.dim() < 1:
        raise RuntimeError("quantize_fp8_row: input must have at least one dimension")
    if a.dim() > 4:
        # same restriction as the reference's GPU path (fp8_quantize.py:235: "Only up to 4 dimension input tensor is supported")
        raise RuntimeError("Only up to 4 dimension input tensor is supported if use_triton is True")
    K = a.shape[-1]
    if K == 0:
        raise RuntimeError("quantize_fp8_row: cannot take the row maximum of an empty last dimension")
    lead = a.shape[:-1]
    rows = 1
    for d in lead:
        rows *= d
    # The kernel takes one row stride; anything else (transposed views, broadcast dims) is packed first.
    if a.stride(-1) == 1 and a.dim() == 2:
        a2, row_stride = a, a.stride(0)
    elif a.is_contiguous():
        a2, row_stride = a, K
    else:
        a2, row_stride = a.contiguous(), K
    K_out = K
    if align_rows_to is not None:
        K_out = (K + align_rows_to - 1) // align_rows_to * align_rows_to
    xq = torch.empty(lead + (K_out,), dtype=FP8_DTYPE, device=a.device)
    scale = torch.empty(lead, dtype=torch.float32, device=a.device)
    ub_ptr = None
    if scale_ub is not None:
        if scale_ub.device != a.device:
            raise RuntimeError("'scale_ub' must be on the same device as 'a'")   # fp8_quantize.py:229-230
        scale_ub = scale_ub.to(dtype=torch.float32).reshape(-1)[:1].contiguous()
        ub_ptr = scale_ub.data_ptr()
    zs_ptr, zs_code, rows_per_group = None, 0, 1
    if zero_start_index_M is not None:
        # One entry per [N, K] matrix of the input viewed as [B, M, N, K] (fp8_quantize.py:236-243).
        rows_per_group = a.shape[-2] if a.dim() >= 2 else 1
        zs = zero_start_index_M
        if zs.device != a.device:
            raise RuntimeError("'zero_start_index_M' must be on the same device as 'a'")
        if zs.dtype not in (torch.int64, torch.int32):
            raise RuntimeError(f"zero_start_index_M must be int64 or int32, got {zs.dtype}")
        if rows_per_group == 0 or zs.numel() * rows_per_group != rows:
            raise RuntimeError(f"zero_start_index_M must have one entry per group of {rows_per_group} rows "
                               f"({rows // max(rows_per_group, 1)} entries), got {zs.numel()}")
        zs = zs.contiguous()
        zs_ptr, zs_code = zs.data_ptr(), (0 if zs.dtype == torch.int64 else 1)
    if rows == 0:
        return xq, scale
    with _on_device(a.device):
        if triton_eps is not None:
            _lib.check(_lib.lib().mslk_amd_quantize_fp8_row_triton_arithmetic(
                a2.data_ptr(), _DTYPE_CODE[a.dtype], rows, K, row_stride, xq.data_ptr(), K_out, scale.data_ptr(), ub_ptr,
                float(triton_eps), zs_ptr, zs_code, rows_per_group, _stream_ptr(a.device)))
        elif zs_ptr is not None:
            _lib.check(_lib.lib().mslk_amd_quantize_fp8_row_jagged(
                a2.data_ptr(), _DTYPE_CODE[a.dtype], rows, K, row_stride, xq.data_ptr(), K_out,
                scale.data_ptr(), ub_ptr, zs_ptr, zs_code, rows_per_group, _stream_ptr(a.device)))
        else:
            _lib.check(_lib.lib().mslk_amd_quantize_fp8_row(
                a2.data_ptr(), _DTYPE_CODE[a.dtype], rows, K, row_stride, xq.data_ptr(), K_out,
                scale.data_ptr(), ub_ptr, _stream_ptr(a.device)))
    return xq, scale


# Lower bound of amax when the caller passes eps_opt=None: get_fp8_constants()'s eps (mslk/utils/triton/fp8_utils.py:23-40).
_FP8_EPS = 1e-12


def _quantize_fp8_row_gpu(a, scale_ub=None, zero_start_index_M=None, use_triton=True, output_device=None,
                          align_rows_to=None, eps_opt=1.0 / 512.0):
    """GPU kernel of `triton::quantize_fp8_row` (reference: fp8_quantize.py:319-378).  As in the reference, `use_triton`
    picks the arithmetic: True = its GPU (Triton) kernel's -- amax clamped at `eps_opt`, scale = amax / 448,
    code = clamp(x / scale, +-448), saturating (131-207) -- False = its torch branch's -- amax clamped at 1e-12 in the input
    dtype, inv = (1 / amax) * 448, code = cast(x * inv) without saturation, scale = 1 / inv (356-378).  The torch branch of
    the reference ignores `zero_start_index_M` and `align_rows_to`; here both arithmetics honour them."""
    triton_eps = None
    if use_triton:
        triton_eps = eps_opt if eps_opt is not None else _FP8_EPS
    a_fp8, a_scale = _quantize_launch(a, scale_ub, zero_start_index_M, align_rows_to, triton_eps)
    if output_device is not None and torch.device(output_device) != a.device:
        a_fp8, a_scale = a_fp8.to(output_device), a_scale.to(output_device)
    return a_fp8, a_scale


def _quantize_fp8_row_fake(a, scale_ub=None, zero_start_index_M=None, use_triton=True, output_device=None,
                           align_rows_to=None, eps_opt=1.0 / 512.0):
    # shape function of the reference (fp8_quantize.py:381-407)
    dev = a.device if output_device is None else output_device
    K = a.shape[-1]
    if align_rows_to is not None:
        K = (K + align_rows_to - 1) // align_rows_to * align_rows_to
    return (torch.empty(tuple(a.shape[:-1]) + (K,), dtype=FP8_DTYPE, device=dev),
            torch.empty(a.shape[:-1], dtype=torch.float32, device=dev))


def _quantize_fp8_per_row_gpu(input, bs=None, scale_ub=None, output_dtype=None, stochastic_rounding=False):
    """GPU kernel of `mslk::quantize_fp8_per_row` (a convenience operator, not one of the reference's): row amax,
    scale = amax / 448, cast to e4m3fn, with the bits of the reference's torch emulation (fp8_quantize.py:356-378)."""
    if bs is not None:
        raise NotImplementedError("quantize_fp8_per_row: `bs` is not supported")
    if stochastic_rounding:
        raise NotImplementedError("quantize_fp8_per_row: stochastic rounding is not supported")
    if output_dtype is not None and output_dtype != FP8_DTYPE:
        raise RuntimeError(f"quantize_fp8_per_row: only {FP8_DTYPE} output is supported on gfx950")
    return _quantize_launch(input, scale_ub, None, None, None)


def _quantize_fp8_per_row_fake(input, bs=None, scale_ub=None, output_dtype=None, stochastic_rounding=False):
    return (torch.empty(input.shape, dtype=FP8_DTYPE, device=input.device),
            torch.empty(input.shape[:-1], dtype=torch.float32, device=input.device))


# Registered with the low-level library API (a few microseconds of dispatch per call); GPU kernels only.
# `triton::quantize_fp8_row` is the operator the reference's torch.library.custom_op (fp8_quantize.py:319-328) defines,
# with its schema and defaults, so a traced or compiled caller of torch.ops.triton.quantize_fp8_row lands here.  When the
# reference defined the op first, only its GPU kernel is replaced; the other way round does not work (the reference's
# custom_op would meet an existing definition), so a process that uses both imports the reference's module first.
# `mslk::quantize_fp8_per_row` has no counterpart in the reference tree: it is a convenience operator under the name the
# path is known by (the legacy FBGEMM operator's signature), always with the torch branch's arithmetic.
_library = torch.library.Library("mslk", "FRAGMENT")
_triton_library = torch.library.Library("triton", "FRAGMENT")
_QUANTIZE_ROW_SCHEMA = ("quantize_fp8_row(Tensor a, Tensor? scale_ub=None, Tensor? zero_start_index_M=None, "
                        "bool use_triton=True, Device? output_device=None, SymInt? align_rows_to=None, "
                        "float? eps_opt=0.001953125) -> (Tensor, Tensor)")
_QUANTIZE_PER_ROW_SCHEMA = ("quantize_fp8_per_row(Tensor input, Tensor? bs=None, Tensor? scale_ub=None, "
                            "ScalarType? output_dtype=None, bool stochastic_rounding=False) -> (Tensor, Tensor)")


def _register_quantize() -> None:
    if hasattr(torch.ops.triton, "quantize_fp8_row"):
        _triton_library.impl("quantize_fp8_row", _quantize_fp8_row_gpu, "CUDA", allow_override=True)
    else:
        _triton_library.define(_QUANTIZE_ROW_SCHEMA)
        _triton_library.impl("quantize_fp8_row", _quantize_fp8_row_gpu, "CUDA")
        torch.library.register_fake("triton::quantize_fp8_row", _quantize_fp8_row_fake, lib=_triton_library)
    if hasattr(torch.ops.mslk, "quantize_fp8_per_row"):
        _library.impl("quantize_fp8_per_row", _quantize_fp8_per_row_gpu, "CUDA", allow_override=True)
    else:
        _library.define(_QUANTIZE_PER_ROW_SCHEMA)
        _library.impl("quantize_fp8_per_row", _quantize_fp8_per_row_gpu, "CUDA")
        torch.library.register_fake("mslk::quantize_fp8_per_row", _quantize_fp8_per_row_fake, lib=_library)


_register_quantize()


def quantize_fp8_row(
    a: torch.Tensor,
    scale_ub: Optional[torch.Tensor] = None,
    zero_start_index_M: Optional[torch.Tensor] = None,
    use_triton: bool = True,
    output_device: Optional[torch.device] = None,
    align_rows_to: Optional[int] = None,
    eps_opt: Optional[float] = 1.0 / 512.0,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Quantize `a` to e4m3fn with one fp32 scale per row (reference signature and dispatch, fp8_quantize.py:319-378).

    Returns (a_fp8 with a's shape [last dim padded to align_rows_to], scale with shape a.shape[:-1]).
    `use_triton=True` (the default, as in the reference) gives the arithmetic of the reference's GPU kernel: amax
    clamped at `eps_opt` (and `scale_ub`), scale = amax / 448, codes = clamp(a / scale, +-448).  `use_triton=False` gives
    the bits of the reference's torch emulation -- the contract this build is checked against bit for bit: amax clamped
    at 1e-12 in the input dtype, inv = (1 / amax) * 448, codes = cast(a * inv) (values beyond 464 become NaN codes,
    which only happens when `scale_ub` cuts the row maximum), scale = 1 / inv; `eps_opt` has no effect there.
    With `zero_start_index_M` (one entry per [N, K] matrix of the input viewed as [B, M, N, K]) the rows
    n >= zero_start_index_M[b, m] are not read and quantize like all-zero rows (fp8_quantize.py:123-129).
    The input must live on a GPU: there is no CPU implementation in this package.
    """
    if not a.is_cuda:
        raise RuntimeError("mslk_amd.quantize_fp8_row: input must be a GPU tensor (no CPU implementation)")
    return torch.ops.triton.quantize_fp8_row(a, scale_ub, zero_start_index_M, use_triton, output_device, align_rows_to,
                                             eps_opt)


def _dequantize_impl(xq: torch.Tensor, x_scale: torch.Tensor) -> torch.Tensor:
    if not (xq.is_contiguous() and x_scale.is_contiguous()):
        raise RuntimeError("Input tensors must be contiguous")
    if xq.dtype != FP8_DTYPE:
        raise RuntimeError(f"dequantize_fp8_row: xq must be {FP8_DTYPE}, got {xq.dtype}")
    if x_scale.dtype != torch.float32 or x_scale.device != xq.device:
        raise RuntimeError("dequantize_fp8_row: x_scale must be a float32 tensor on the device of xq")
    if xq.dim() < 1:
        raise RuntimeError("dequantize_fp8_row: xq must have at least one dimension")
    K = xq.shape[-1]
    rows = xq.numel() // K if K else 0
    if x_scale.numel() != (rows if K else x_scale.numel()):
        raise RuntimeError(f"dequantize_fp8_row: x_scale must have one entry per row ({rows}), got {x_scale.numel()}")
    out = torch.empty(xq.shape, dtype=torch.bfloat16, device=xq.device)
    if rows > 0:
        with _on_device(xq.device):
            _lib.check(_lib.lib().mslk_amd_dequantize_fp8_row(xq.data_ptr(), x_scale.data_ptr(), rows, K, out.data_ptr(),
                                                              _stream_ptr(xq.device)))
    return out


if not hasattr(torch.ops.mslk, "dequantize_fp8_row"):
    _library.define("dequantize_fp8_row(Tensor xq, Tensor x_scale) -> Tensor")
    _library.impl("dequantize_fp8_row", _dequantize_impl, "CUDA")
    torch.library.register_fake(
        "mslk::dequantize_fp8_row",
        lambda xq, x_scale: torch.empty(xq.shape, dtype=torch.bfloat16, device=xq.device), lib=_library)


def dequantize_fp8_row(xq: torch.Tensor, x_scale: torch.Tensor) -> torch.Tensor:
    """Row-wise dequantization to bf16 along the last axis (reference signature, fp8_quantize.py:1140-1182):
    out = bf16(float(xq) * x_scale[..., None]), the product taken in fp32."""
    if not xq.is_cuda:
        raise RuntimeError("mslk_amd.dequantize_fp8_row: input must be a GPU tensor (no CPU implementation)")
    return torch.ops.mslk.dequantize_fp8_row(xq, x_scale)


def quantize_fp8_per_row(
    input: torch.Tensor,
    bs: Optional[torch.Tensor] = None,
    scale_ub: Optional[torch.Tensor] = None,
    output_dtype: Optional[torch.dtype] = None,
    stochastic_rounding: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row amax -> scale = amax / 448 -> e4m3fn codes, bit-exact to the reference's torch emulation
    (`quantize_fp8_row(..., use_triton=False)`, fp8_quantize.py:356-378); the legacy operator name of the path (the
    reference's bench still calls it `CudaFP8Rowwise`, bench/quantize/quantize_ops.py:242-251).  `bs` and stochastic
    rounding are not supported."""
    if not input.is_cuda:
        raise RuntimeError("mslk_amd.quantize_fp8_per_row: input must be a GPU tensor (no CPU implementation)")
    return torch.ops.mslk.quantize_fp8_per_row(input, bs, scale_ub, output_dtype, stochastic_rounding)
