"""torch.library.opcheck on the registered ops: the fake (meta) kernels agree with the real ones in shape, dtype,
strides and device (the reference registers fake kernels
for the same purpose, mslk/gemm/_meta.py:26-65,114-126 and mslk/quantize/triton/fp8_quantize.py:381-407)."""
import pytest
import torch

import mslk_amd  # noqa: F401
from mslk_amd import moe  # noqa: F401

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn
CHECKS = ("test_faketensor",)   # the schema checker multiplies tensors, which float8 does not implement


def _codes(*shape):
    return torch.randint(0, 0x58, shape, dtype=torch.uint8, device=DEV).view(F8)


def test_opcheck_quantize_and_dequantize():
    x = torch.randn(48, 256, device=DEV, dtype=torch.bfloat16)
    torch.library.opcheck(torch.ops.triton.quantize_fp8_row, (x,), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.mslk.quantize_fp8_per_row, (x,), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.triton.quantize_fp8_row, (x, torch.tensor([1200.0], device=DEV), None, False, None, 64),
                          test_utils=CHECKS)
    q, s = torch.ops.triton.quantize_fp8_row(x)
    torch.library.opcheck(torch.ops.mslk.dequantize_fp8_row, (q, s), test_utils=CHECKS)


def test_opcheck_quantize_fused_gemm():
    x = torch.randn(5, 2048, device=DEV, dtype=torch.bfloat16)
    torch.library.opcheck(torch.ops.mslk.quantize_f8f8bf16_rowwise, (x, _codes(96, 2048), torch.rand(96, device=DEV) + 0.5),
                          test_utils=CHECKS)
    x = torch.randn(40, 256, device=DEV, dtype=torch.bfloat16)       # two-launch shape
    torch.library.opcheck(torch.ops.mslk.quantize_f8f8bf16_rowwise,
                          (x, _codes(96, 256), torch.rand(96, device=DEV) + 0.5, torch.randn(96, device=DEV)), test_utils=CHECKS)


def test_opcheck_dense_family():
    M, N, K = 80, 96, 256
    xq, wq = _codes(M, K), _codes(N, K)
    xs, ws = torch.rand(M, device=DEV) + 0.5, torch.rand(N, device=DEV) + 0.5
    bias = torch.randn(N, device=DEV)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise, (xq, wq, xs, ws), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise, (xq, wq, xs, ws, bias), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.mslk.f8f8f16_rowwise, (xq, wq, xs, ws), test_utils=CHECKS)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_out, (xq, wq, xs, ws, out), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_batched,
                          (_codes(3, M, K), _codes(3, N, K), torch.rand(3, M, device=DEV), torch.rand(3, N, device=DEV)),
                          test_utils=CHECKS)


def test_opcheck_grouped_family():
    G, N, K = 3, 64, 128
    sizes = [5, 0, 40]
    M = sum(sizes)
    xq, wq = _codes(M, K), _codes(G, N, K)
    xs, ws = torch.rand(M, device=DEV) + 0.5, torch.rand(G, N, device=DEV) + 0.5
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked,
                          (xq, wq, xs, ws, torch.tensor(sizes, dtype=torch.int64, device=DEV)), test_utils=CHECKS)
    ends = torch.tensor(sizes, device=DEV).cumsum(0).to(torch.int32)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)   # the reference's schema takes the output tensor
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_grouped_mm, (xq, wq, xs, ws, ends, out), test_utils=CHECKS)
    # the TensorList op keeps the reference's check that N and K are at least 512
    xq2, wq2 = _codes(M, 512), _codes(G, 512, 512)
    ws2 = torch.rand(G, 512, device=DEV) + 0.5
    xl, sl = list(xq2.split(sizes)), list(xs.split(sizes))
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_grouped, (xl, list(wq2), sl, list(ws2)), test_utils=CHECKS)


def test_opcheck_fused_producers():
    T, D, E = 24, 256, 4
    x = torch.randn(T, 2 * D, device=DEV, dtype=torch.bfloat16)
    torch.library.opcheck(torch.ops.mslk.silu_mul_quant, (x[:, :D], x[:, D:]), test_utils=CHECKS)
    tok = torch.randperm(T, device=DEV).to(torch.int32)
    exp = torch.randint(0, E, (T,), device=DEV)
    scores = torch.rand(T, E, device=DEV)
    torch.library.opcheck(torch.ops.mslk.gather_scale_quant_dense_tokens, (x[:, :D].contiguous(), tok, exp, scores),
                          test_utils=CHECKS)


def test_opcheck_preshuffle_dynamic_and_cat():
    M, N, K = 48, 64, 128
    xq, wq = _codes(M, K), _codes(N, K)
    xs, ws = torch.rand(M, device=DEV) + 0.5, torch.rand(N, device=DEV) + 0.5
    wps = mslk_amd.preshuffle_b_mfma(wq)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_preshuffle, (xq, wps, xs, ws), test_utils=CHECKS)
    torch.library.opcheck(torch.ops.mslk.f8f8f16_rowwise_preshuffle, (xq, wps, xs, ws), test_utils=CHECKS)
    G = 3
    xq3, wq3 = _codes(G, M, 512), _codes(G, 512, 512)          # the reference's check: N and K at least 512
    xs3, ws3 = torch.rand(G, M, device=DEV) + 0.5, torch.rand(G, 512, device=DEV) + 0.5
    live = torch.tensor([5, 0, 48], dtype=torch.int64, device=DEV)
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_grouped_dynamic, (xq3, wq3, xs3, ws3, live), test_utils=CHECKS)
    sizes = [5, 0, 40]
    xq2, wq2 = _codes(sum(sizes), 512), _codes(G, 512, 512)
    xs2, ws2 = torch.rand(sum(sizes), device=DEV) + 0.5, torch.rand(G, 512, device=DEV) + 0.5
    torch.library.opcheck(torch.ops.mslk.f8f8bf16_rowwise_grouped_cat,
                          (list(xq2.split(sizes)), list(wq2), list(xs2.split(sizes)), list(ws2)), test_utils=CHECKS)


def test_ops_trace_under_torch_compile():
    """Dynamo + AOT autograd with fake tensors trace quantize -> GEMM into one graph (no graph breaks) and the compiled
    function returns what the eager one does."""
    w = torch.randn(96, 256, device=DEV, dtype=torch.bfloat16)
    wq, ws = mslk_amd.quantize_fp8_row(w)

    def linear(x):
        xq, xs = torch.ops.triton.quantize_fp8_row(x)
        return torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)

    x = torch.randn(40, 256, device=DEV, dtype=torch.bfloat16)
    compiled = torch.compile(linear, backend="aot_eager", fullgraph=True)
    assert torch.equal(compiled(x), linear(x))
