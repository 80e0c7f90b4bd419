"""Fused producers of the FP8 activations of the MoE GEMMs, behind the reference's Python interface.

`silu_mul_quant` (mslk/moe/activation.py:72-135) and `gather_scale_quant_dense_tokens`
(mslk/moe/gather_scatter.py:96-170) keep the reference's signatures and are also registered as
`torch.ops.mslk.silu_mul_quant` / `torch.ops.mslk.gather_scale_quant_dense_tokens` (GPU kernels
only).  The second op's schema declares the tuple it really returns (the reference's schema string
says `-> Tensor` while its kernels return two tensors).
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .quantize import FP8_DTYPE, _on_device, _stream_ptr

_X_DTYPE = {torch.bfloat16: 0, torch.float16: 1}
_SCORE_DTYPE = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
_INDEX_DTYPE = {torch.int64: 0, torch.int32: 1}


def _check(cond: bool, msg: str) -> None:
    if not cond:
        raise RuntimeError(msg)


def _optional_scalars(scale_ub, valid_token_count, device):
    ub_ptr, keep_ub = None, None
    if scale_ub is not None:
        keep_ub = scale_ub.to(device=device, dtype=torch.float32).reshape(-1)[:1].contiguous()
        ub_ptr = keep_ub.data_ptr()
    cnt_ptr, cnt_code = None, 0
    if valid_token_count is not None:
        _check(valid_token_count.device == device, "valid_token_count must be on the device of the inputs")
        _check(valid_token_count.dtype in _INDEX_DTYPE, "valid_token_count must be int32 or int64")
        _check(valid_token_count.numel() >= 1, "valid_token_count must hold one element")
        cnt_ptr, cnt_code = valid_token_count.data_ptr(), _INDEX_DTYPE[valid_token_count.dtype]
    return ub_ptr, keep_ub, cnt_ptr, cnt_code


def _silu_mul_quant_impl(x0: torch.Tensor, x1: torch.Tensor, scale_ub: Optional[torch.Tensor] = None,
                         valid_token_count: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    _check(x0.dim() == 2 and x0.stride(1) == 1, "x0 must be 2-D with unit column stride")
    _check(x1.dim() == 2 and x1.stride(1) == 1, "x1 must be 2-D with unit column stride")
    _check(x0.shape == x1.shape, "x0 and x1 must have the same shape")
    _check(x0.dtype == x1.dtype, "x0 and x1 must have the same dtype")
    _check(x0.dtype in _X_DTYPE, f"silu_mul_quant: inputs must be bfloat16 or float16, got {x0.dtype}")
    _check(x1.device == x0.device, "x0 and x1 must be on the same device")
    T, D = x0.shape
    out = torch.empty((T, D), device=x0.device, dtype=FP8_DTYPE)
    out_scale = torch.empty((T,), device=x0.device, dtype=torch.float32)
    if T == 0 or D == 0:
        return out, out_scale
    ub_ptr, _keep, cnt_ptr, cnt_code = _optional_scalars(scale_ub, valid_token_count, x0.device)
    with _on_device(x0.device):
        _lib.check(_lib.lib().mslk_amd_silu_mul_quant(
            x0.data_ptr(), x1.data_ptr(), _X_DTYPE[x0.dtype], T, D, x0.stride(0), x1.stride(0), out.data_ptr(),
            out_scale.data_ptr(), ub_ptr, cnt_ptr, cnt_code, _stream_ptr(x0.device)))
    return out, out_scale


def _gather_scale_quant_impl(x: torch.Tensor, token_indices: torch.Tensor, expert_indices: torch.Tensor,
                             scores: torch.Tensor, scale_ub: Optional[torch.Tensor] = None,
                             valid_token_count: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    _check(x.dim() == 2 and x.is_contiguous(), "x must be a contiguous 2-D tensor")
    _check(token_indices.is_contiguous() and expert_indices.is_contiguous(), "index tensors must be contiguous")
    T, D = x.shape
    a = token_indices.shape[0]
    _check(tuple(token_indices.shape) == (a,) and tuple(expert_indices.shape) == (a,), "index tensors must have shape (a,)")
    _check(scores.dim() == 2 and scores.shape[0] == T, "scores must have shape (T, E)")
    E = scores.shape[1]
    _check(x.dtype in _X_DTYPE, f"gather_scale_quant_dense_tokens: x must be bfloat16 or float16, got {x.dtype}")
    _check(scores.dtype in _SCORE_DTYPE, f"scores must be bfloat16, float16 or float32, got {scores.dtype}")
    _check(token_indices.dtype in _INDEX_DTYPE and expert_indices.dtype in _INDEX_DTYPE, "indices must be int32 or int64")
    _check(token_indices.device == x.device and expert_indices.device == x.device and scores.device == x.device,
           "all operands must be on the same device")
    out = torch.empty((a, D), device=x.device, dtype=FP8_DTYPE)
    out_scale = torch.empty((a,), device=x.device, dtype=torch.float32)
    if a == 0 or D == 0:
        return out, out_scale
    ub_ptr, _keep, cnt_ptr, cnt_code = _optional_scalars(scale_ub, valid_token_count, x.device)
    with _on_device(x.device):
        _lib.check(_lib.lib().mslk_amd_gather_scale_quant_dense_tokens(
            x.data_ptr(), _X_DTYPE[x.dtype], T, D, token_indices.data_ptr(), _INDEX_DTYPE[token_indices.dtype],
            expert_indices.data_ptr(), _INDEX_DTYPE[expert_indices.dtype], a, scores.data_ptr(),
            _SCORE_DTYPE[scores.dtype], E, scores.stride(0), scores.stride(1), out.data_ptr(), out_scale.data_ptr(),
            ub_ptr, cnt_ptr, cnt_code, _stream_ptr(x.device)))
    return out, out_scale


def _fake_silu_mul_quant(x0, x1, scale_ub=None, valid_token_count=None):
    return (torch.empty(x0.shape, device=x0.device, dtype=FP8_DTYPE),
            torch.empty((x0.shape[0],), device=x0.device, dtype=torch.float32))


def _fake_gather_scale_quant(x, token_indices, expert_indices, scores, scale_ub=None, valid_token_count=None):
    # mslk/moe/gather_scatter.py:331-345
    a, D = token_indices.shape[0], x.shape[1]
    return (torch.empty((a, D), device=x.device, dtype=FP8_DTYPE), torch.empty((a,), device=x.device, dtype=torch.float32))


_library = torch.library.Library("mslk", "FRAGMENT")
_OPS = {
    "silu_mul_quant": ("(Tensor x0, Tensor x1, Tensor? scale_ub=None, Tensor? valid_token_count=None) -> (Tensor, Tensor)",
                       _silu_mul_quant_impl, _fake_silu_mul_quant),
    "gather_scale_quant_dense_tokens": (
        "(Tensor x, Tensor token_indices, Tensor expert_indices, Tensor scores, Tensor? scale_ub=None, "
        "Tensor? valid_token_count=None) -> (Tensor, Tensor)", _gather_scale_quant_impl, _fake_gather_scale_quant),
}
for _name, (_schema, _impl, _fake) in _OPS.items():
    if hasattr(torch.ops.mslk, _name):
        _library.impl(_name, _impl, "CUDA", allow_override=True)
    else:
        _library.define(_name + _schema)
        _library.impl(_name, _impl, "CUDA")
        torch.library.register_fake(f"mslk::{_name}", _fake, lib=_library)


def silu_mul_quant(x0: torch.Tensor, x1: torch.Tensor, scale_ub: Optional[torch.Tensor] = None,
                   valid_token_count: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """y, y_scale = quantize(x0 * sigmoid(x0) * x1) for x0, x1 of shape (T, D); rows at or beyond
    valid_token_count[0] are left uninitialised (reference signature, mslk/moe/activation.py:72-93)."""
    if not x0.is_cuda:
        raise RuntimeError("mslk_amd.silu_mul_quant: inputs must be GPU tensors (no CPU implementation)")
    return torch.ops.mslk.silu_mul_quant(x0, x1, scale_ub, valid_token_count)


def gather_scale_quant_dense_tokens(x: torch.Tensor, token_indices: torch.Tensor, expert_indices: torch.Tensor,
                                    scores: torch.Tensor, scale_ub: Optional[torch.Tensor] = None,
                                    valid_token_count: Optional[torch.Tensor] = None
                                    ) -> Tuple[torch.Tensor, torch.Tensor]:
    """out[i] = quantize(x[token_indices[i]] * scores[token_indices[i], expert_indices[i]])
    (reference signature, mslk/moe/gather_scatter.py:96-128)."""
    if not x.is_cuda:
        raise RuntimeError("mslk_amd.gather_scale_quant_dense_tokens: inputs must be GPU tensors (no CPU implementation)")
    return torch.ops.mslk.gather_scale_quant_dense_tokens(x, token_indices, expert_indices, scores, scale_ub,
                                                          valid_token_count)
