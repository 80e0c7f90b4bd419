"""CPU oracle for the FP8 rowwise quantized-linear path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import this
module.  The product package (mslk_amd) never imports it and has no CPU fallback.

Every function restates, in plain CPU torch, the arithmetic of one reference function
(paths relative to the reference checkout):

  quantize_fp8_row        mslk/quantize/triton/fp8_quantize.py:356-378  (torch branch)
  fp8 constants           mslk/utils/triton/fp8_utils.py:23-40          (e4m3fn, 448.0, 1e-12)
  dequant_matmul          test/gemm/triton/fp8_gemm_test.py:126-132     (tight GEMM oracle)
  matmul_fp8_row_cpu      mslk/gemm/triton/fp8_gemm.py:1186-1201        (CPU fallback = timed CPU baseline)
  grouped_*               test/gemm/triton/grouped_gemm_test.py:116-121, bench/gemm/gemm_ops.py:632-644
  quantize_fp8_row_triton_arithmetic  mslk/quantize/triton/fp8_quantize.py:131-207 (parity unpinned at bit
                          level: the Triton kernel cannot run here; closed forms only)
  quantize_fp8_row_jagged mslk/quantize/triton/fp8_quantize.py:123-129,236-243
  dequantize_fp8_row[_bf16] mslk/quantize/triton/fp8_quantize.py:1060-1113
  preshuffle_b            mslk/quantize/shuffle.py:182-246
  quantize_rows_saturating, silu_mul_quant, gather_scale_quant_dense_tokens
                          mslk/moe/activation.py:232-300, mslk/moe/gather_scatter.py:545-640

Pinning (what keeps this file honest; see tests/test_oracle.py):
  * quantize: the scalar C twin in oracle/fp8_rowwise_oracle.c shares no code with torch and is
    compared bit-for-bit, exhaustively over all 65536 bf16 inputs for many row maxima; closed
    forms (amax = 448*2^k, zero rows, one-hot rows, -0.0, NaN rows) are asserted separately.
  * dequant_matmul: brute-force float64 triple loop (C twin), identity / one-hot weights,
    integer-valued codes where fp32 accumulation is exact.
  * jagged / dequantize / saturating quantization: closed forms and hand-worked roundings.
  * silu_mul_quant: the sigmoid is torch's CPU sigmoid; the reference's Triton sigmoid may differ in
    the last bits, so parity is unpinned at bit level and held to the reference test's own
    tolerance (test/moe/activation_test.py:168-170) plus a bound on the fraction of differing codes.
  * matmul_fp8_row_cpu: parity unpinned at bit level (it is a timing baseline whose bf16 matmul
    rounds before scaling); it is only checked to agree with dequant_matmul within bf16 tolerance.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

FP8_DTYPE = torch.float8_e4m3fn  # gfx950 uses OCP e4m3fn (mslk/utils/device.py:135-160)
FP8_MAX = 448.0                  # torch.finfo(float8_e4m3fn).max (fp8_utils.py:40)
EPS = 1e-12                      # fp8_utils.py:40


def quantize_fp8_row(a: torch.Tensor, scale_ub: Optional[torch.Tensor] = None
                     ) -> Tuple[torch.Tensor, torch.Tensor]:
    """fp8_quantize.py:360-378, CPU tensors only.

    row_max is taken and clamped in the INPUT dtype (line 363-369), `448 / t` is
    Tensor.__rdiv__ = t.reciprocal() * 448 (line 371), inf -> 1.0 (372), the product
    a * a_scale is fp32 by type promotion (373), the cast is round-to-nearest-even with
    no saturation (375) and the returned scale is 1 / a_scale = a_scale.reciprocal() (378).
    """
    assert a.device.type == "cpu"
    a_shape = a.shape
    row_max = torch.max(torch.abs(a), dim=-1)[0]
    if scale_ub is not None:
        row_max = torch.clamp(row_max, min=EPS, max=scale_ub.item())
    else:
        row_max = torch.clamp(row_max, min=EPS)
    a_scale = FP8_MAX / row_max.to(torch.float32)
    a_scale[a_scale == float("inf")] = 1.0
    a_fp8 = (a * a_scale[..., None]).to(FP8_DTYPE)
    return a_fp8, (1 / a_scale).view(a_shape[:-1])


def dequantize_fp8_row(xq: torch.Tensor, x_scale: torch.Tensor) -> torch.Tensor:
    """fp32 dequantization xq * scale[:, None] (fp8_quantize.py:1140-1182 semantics)."""
    return xq.to(torch.float32) * x_scale.to(torch.float32).reshape(*xq.shape[:-1], 1)


def quantize_fp8_row_triton_arithmetic(a: torch.Tensor, scale_ub: Optional[torch.Tensor] = None,
                                       eps: float = 1.0 / 512.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """The arithmetic written in the reference's Triton kernel (fp8_quantize.py:131-207; eps_opt default
    1/512, lines 215,246-247), restated with IEEE fp32 operations:
        amax = clamp(max|a| (taken in a's dtype), eps [, scale_ub]);  scale = amax / 448 (div_rn);
        code = e4m3fn_rne(clamp(a.f32 / scale (div_rn), -448, 448)).
    The Triton kernel itself cannot be executed here, so this restatement is pinned only by closed forms."""
    amax = a.abs().amax(dim=-1).to(torch.float32)
    amax = torch.clamp(amax, min=eps)
    if scale_ub is not None:
        amax = torch.minimum(amax, scale_ub.reshape(-1)[0].to(torch.float32))
    scale = amax / torch.tensor(FP8_MAX, dtype=torch.float32)
    q = torch.clamp(a.to(torch.float32) / scale[..., None], -FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, scale


def dequantize_fp8_row_bf16(xq: torch.Tensor, x_scale: torch.Tensor) -> torch.Tensor:
    """What the reference's dequantize kernel stores (fp8_quantize.py:1096-1112): the fp32 product
    of the decoded code and the row scale, rounded to bf16 (nearest even) by the store."""
    return dequantize_fp8_row(xq, x_scale).to(torch.bfloat16)


def quantize_fp8_row_jagged(a: torch.Tensor, zero_start_index_M: torch.Tensor,
                            scale_ub: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """Jagged variant (fp8_quantize.py:236-243 grouping, 123-129 row rule): with `a` viewed as
    [B, M, N, K] and zero_start_index_M as [B, M], row n of matrix (b, m) is loaded with an empty
    mask when n >= zero_start_index_M[b, m], i.e. it is quantized as a row of zeros."""
    a4 = a
    while a4.dim() < 4:
        a4 = a4.unsqueeze(0)
    zs = zero_start_index_M.reshape(a4.shape[0], a4.shape[1]).to(torch.int64)
    n = torch.arange(a4.shape[2]).reshape(1, 1, -1)
    live = n < zs[:, :, None]
    masked = torch.where(live[..., None], a4, torch.zeros((), dtype=a.dtype)).reshape(a.shape)
    return quantize_fp8_row(masked, scale_ub)


def quantize_rows_saturating(y: torch.Tensor, scale_ub: Optional[torch.Tensor] = None
                             ) -> Tuple[torch.Tensor, torch.Tensor]:
    """Row-wise quantization as written inside the reference's fused MoE kernels
    (mslk/moe/activation.py:281-297, mslk/moe/gather_scatter.py:601-633), all in fp32:
        row_max = clamp(max|y|, 1e-12 [, scale_ub]);  s = 448 / row_max;  scale = 1 / s;
        code = e4m3fn_rne(clamp(y * s, -448, 448)).
    It differs from quantize_fp8_row (the torch branch) in the order of the two divisions and in that
    it saturates instead of producing NaN when scale_ub cuts the maximum."""
    y = y.to(torch.float32)
    row_max = y.abs().amax(dim=-1)
    if scale_ub is not None:
        row_max = torch.clamp(row_max, min=1e-12, max=float(scale_ub.reshape(-1)[0].to(torch.float32)))
    else:
        row_max = torch.clamp(row_max, min=1e-12)
    s = torch.tensor(FP8_MAX, dtype=torch.float32) / row_max
    q = torch.clamp(y * s[..., None], -FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, 1.0 / s


def silu_mul_quant(x0: torch.Tensor, x1: torch.Tensor, scale_ub: Optional[torch.Tensor] = None
                   ) -> Tuple[torch.Tensor, torch.Tensor]:
    """quantize(x0 * sigmoid(x0) * x1), the product taken in fp32 left to right
    (mslk/moe/activation.py:270-279; the same expression is the reference test's own oracle,
    test/moe/activation_test.py:159-163)."""
    a, b = x0.to(torch.float32), x1.to(torch.float32)
    return quantize_rows_saturating(a * torch.sigmoid(a) * b, scale_ub)


def gather_scale_quant_dense_tokens(x: torch.Tensor, token_indices: torch.Tensor, expert_indices: torch.Tensor,
                                    scores: torch.Tensor, scale_ub: Optional[torch.Tensor] = None
                                    ) -> Tuple[torch.Tensor, torch.Tensor]:
    """quantize(x[token] * scores[token, expert]) in fp32 (mslk/moe/gather_scatter.py:564-633; the
    reference test builds the same product, test/moe/gather_scatter_test.py:170-182)."""
    t, e = token_indices.to(torch.int64), expert_indices.to(torch.int64)
    y = x[t].to(torch.float32) * scores[t, e].to(torch.float32)[:, None]
    return quantize_rows_saturating(y, scale_ub)


def preshuffle_b(src: torch.Tensor) -> torch.Tensor:
    """Blocked weight layout of the reference's pre-shuffled GEMMs (mslk/quantize/shuffle.py:182-246):
    the trailing [N, K] is cut into 16-row x 64-column blocks, (N/16, 16, K/64, 4, 16), and stored in
    the order (N/16, K/64, 4, 16, 16) -- block, 16-byte k chunk, row, byte.  Same shape as src."""
    N, K = src.shape[-2], src.shape[-1]
    assert N % 16 == 0 and K % 64 == 0
    lead = src.shape[:-2]
    v = src.reshape(*lead, N // 16, 16, K // 64, 4, 16)
    nd = v.dim()
    v = v.permute(*range(nd - 5), nd - 5, nd - 3, nd - 2, nd - 4, nd - 1).contiguous()
    return v.reshape(*lead, N, K)


def dequant_matmul(xq: torch.Tensor, wq: torch.Tensor, x_scale: torch.Tensor,
                   w_scale: torch.Tensor, bias: Optional[torch.Tensor] = None,
                   dtype: torch.dtype = torch.float32) -> torch.Tensor:
    """(xq.f32 * xs[:, None]) @ (wq.f32 * ws[:, None]).T [+ bias.f32]; no output rounding.

    Same expression as test/gemm/triton/fp8_gemm_test.py:128-132.  `dtype=torch.float64`
    gives the exact-arithmetic variant used for error budgeting.
    """
    x = xq.reshape(-1, xq.shape[-1]).to(dtype) * x_scale.reshape(-1, 1).to(dtype)
    w = wq.to(dtype) * w_scale.reshape(-1, 1).to(dtype)
    y = x @ w.T
    if bias is not None:
        y = y + bias.to(dtype)[None, :]
    return y.reshape(*xq.shape[:-1], wq.shape[0])


def matmul_fp8_row_cpu(xq: torch.Tensor, wq: torch.Tensor, x_scale: torch.Tensor,
                       w_scale: torch.Tensor, bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """fp8_gemm.py:1186-1201: bf16 matmul, then scale outer product, then bias, then bf16."""
    a = xq.reshape(-1, xq.shape[-1])
    out_shape = tuple(xq.shape[:-1]) + (wq.shape[0],)
    if a.shape[0] == 0 or wq.shape[0] == 0 or a.shape[1] == 0:
        return torch.zeros(out_shape, dtype=torch.bfloat16)
    scale = x_scale.reshape(-1)[:, None] * w_scale[None, :]
    out = torch.matmul(a.to(torch.bfloat16), wq.to(torch.bfloat16).T) * scale
    if bias is not None:
        out += bias[None, :]
    return out.to(torch.bfloat16).reshape(out_shape)


def grouped_dequant_matmul(xq: Sequence[torch.Tensor], wq: Sequence[torch.Tensor],
                           x_scale: Sequence[torch.Tensor], w_scale: Sequence[torch.Tensor]
                           ) -> List[torch.Tensor]:
    """Per-group dequant_matmul (grouped_gemm_test.py:116-121 written as a loop)."""
    return [dequant_matmul(a, b, sa, sb) for a, b, sa, sb in zip(xq, wq, x_scale, w_scale)]


def grouped_matmul_fp8_row_cpu(xq, wq, x_scale, w_scale) -> List[torch.Tensor]:
    """Loop of the CPU fallback over experts (bench/gemm/gemm_ops.py:632-644 pattern)."""
    return [matmul_fp8_row_cpu(a, b, sa, sb) for a, b, sa, sb in zip(xq, wq, x_scale, w_scale)]


# ----------------------------------------------------------------------------------------
# error metrics used by every GEMM parity test (north_star: max-rel 1e-2, normwise 2e-3)
# ----------------------------------------------------------------------------------------
MAX_REL_TOL = 1e-2
NORMWISE_TOL = 2e-3
# elementwise criterion, as the reference's own tests compare (test/gemm/gemm_test.py:493-505,
# test/gemm/triton/fp8_gemm_test.py:128-142), at the tolerance of the path: |y - ref| <= ELEM_RTOL * |ref| + ELEM_ATOL_RMS * rms(ref)
ELEM_RTOL = 1e-2
ELEM_ATOL_RMS = 1e-2


def gemm_errors(y: torch.Tensor, ref: torch.Tensor) -> Tuple[float, float]:
    """(max|y-ref| / max|ref|, ||y-ref||_F / ||ref||_F) in float64."""
    y64 = y.detach().cpu().to(torch.float64)
    r64 = ref.detach().cpu().to(torch.float64)
    if r64.numel() == 0:
        return 0.0, 0.0
    diff = (y64 - r64)
    denom_max = r64.abs().max().item()
    denom_f = torch.linalg.vector_norm(r64).item()
    max_rel = diff.abs().max().item() / denom_max if denom_max > 0 else diff.abs().max().item()
    normwise = torch.linalg.vector_norm(diff).item() / denom_f if denom_f > 0 else torch.linalg.vector_norm(diff).item()
    return max_rel, normwise


def gemm_elementwise_violations(y: torch.Tensor, ref: torch.Tensor, rms: float = None) -> Tuple[int, float]:
    """Number of elements with |y - ref| > ELEM_RTOL * |ref| + ELEM_ATOL_RMS * rms(ref), and the largest value of
    |y - ref| / (ELEM_RTOL * |ref| + ELEM_ATOL_RMS * rms(ref)) (<= 1 passes).  `rms` overrides rms(ref) when `ref`
    is a block of a larger tensor."""
    y64 = y.detach().cpu().to(torch.float64)
    r64 = ref.detach().cpu().to(torch.float64)
    if r64.numel() == 0:
        return 0, 0.0
    if rms is None:
        rms = torch.sqrt(torch.mean(r64 * r64)).item()
    bound = ELEM_RTOL * r64.abs() + ELEM_ATOL_RMS * rms
    diff = (y64 - r64).abs()
    bad = diff > bound
    worst = (diff / bound.clamp_min(1e-300)).max().item() if rms > 0 else (0.0 if not bad.any() else float("inf"))
    return int(bad.sum().item()), worst
