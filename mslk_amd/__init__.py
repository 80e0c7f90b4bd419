"""mslk_amd: MI355X (gfx950) FP8 rowwise quantized-linear path.

Importing the package registers `torch.ops.mslk.f8f8bf16_rowwise`, `..._rowwise_out`,
`..._rowwise_grouped`, `..._rowwise_grouped_cat`, `..._rowwise_grouped_stacked`,
`..._rowwise_grouped_mm`, `..._rowwise_batched` and
`torch.ops.mslk.quantize_fp8_row` / `dequantize_fp8_row`, all backed by hand-written HIP kernels in libmslk_amd.so.
"""
from . import _lib  # noqa: F401
from .quantize import (quantize_fp8_row, quantize_fp8_per_row, dequantize_fp8_row,  # noqa: F401
                       FP8_DTYPE)  # noqa: F401
from . import gemm  # noqa: F401  (registers torch.ops.mslk.*)
from . import moe  # noqa: F401  (registers torch.ops.mslk.silu_mul_quant / gather_scale_quant_dense_tokens)
from .moe import silu_mul_quant, gather_scale_quant_dense_tokens  # noqa: F401
from .gemm import (f8f8bf16_rowwise, f8f8bf16_rowwise_out, quantize_f8f8bf16_rowwise, f8f8f16_rowwise, f8f8bf16_rowwise_preshuffle,
                   f8f8f16_rowwise_preshuffle, preshuffle_b_mfma, ck_preshuffle, f8f8bf16_rowwise_grouped,  # noqa: F401
                   f8f8bf16_rowwise_grouped_cat, f8f8bf16_rowwise_grouped_stacked,
                   f8f8bf16_rowwise_grouped_mm, f8f8bf16_rowwise_grouped_dynamic,
                   f8f8bf16_rowwise_batched)

__all__ = ["quantize_fp8_row", "quantize_fp8_per_row", "dequantize_fp8_row", "silu_mul_quant", "gather_scale_quant_dense_tokens", "f8f8bf16_rowwise", "f8f8bf16_rowwise_out", "quantize_f8f8bf16_rowwise", "f8f8f16_rowwise", "f8f8bf16_rowwise_preshuffle", "f8f8f16_rowwise_preshuffle", "preshuffle_b_mfma", "ck_preshuffle",
           "f8f8bf16_rowwise_grouped", "f8f8bf16_rowwise_grouped_cat", "f8f8bf16_rowwise_grouped_stacked",
           "f8f8bf16_rowwise_grouped_mm", "f8f8bf16_rowwise_grouped_dynamic", "f8f8bf16_rowwise_batched", "FP8_DTYPE"]
