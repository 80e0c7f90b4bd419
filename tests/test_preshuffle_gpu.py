"""GPU parity of the pre-shuffled-weight GEMMs (f8f8bf16_rowwise_preshuffle, f8f8f16_rowwise_preshuffle)
and of the weight re-layout itself.  The re-layout is a permutation and must match the oracle bit for
bit; the GEMMs are held to the same oracle and tolerance as the plain-layout op, plus bit-exact cases
where fp32 accumulation is exact."""
import pytest
import torch

import mslk_amd
from oracle import fp8_rowwise_oracle as O
from tests.helpers import assert_gemm_close, codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F8 = torch.float8_e4m3fn


@pytest.mark.parametrize("shape", [(16, 64), (48, 192), (4096, 4096), (3, 32, 128), (16, 512, 5120), (528, 2112)])
def test_preshuffle_is_the_reference_permutation(shape):
    g = torch.Generator().manual_seed(sum(shape))
    w = torch.randint(0, 256, shape, generator=g, dtype=torch.uint8).view(F8)
    got = mslk_amd.preshuffle_b_mfma(w.to(DEV))
    torch.cuda.synchronize()
    assert got.shape == w.shape and got.dtype == w.dtype
    assert torch.equal(codes(got), O.preshuffle_b(w.view(torch.uint8)))
    if len(shape) == 2:
        assert torch.equal(codes(mslk_amd.ck_preshuffle(w.to(DEV), 16)), codes(got))
    with pytest.raises(ValueError):
        mslk_amd.preshuffle_b_mfma(torch.zeros(24, 64, dtype=torch.uint8, device=DEV).view(F8))


def _problem(M, N, K, g):
    x = torch.randn(M, K, generator=g).bfloat16()
    w = (torch.randn(N, K, generator=g) * 0.02).bfloat16()
    xq, xs = O.quantize_fp8_row(x)
    wq, ws = O.quantize_fp8_row(w)
    return xq, wq, xs, ws


SHAPES = [
    # dense tiles (256^2 and 128^2), ragged M, N a multiple of 16 only, K tails of 64, skinny M with and without K % 1024
    (4096, 4096, 4096), (1024, 1024, 1024), (300, 528, 640), (257, 272, 384), (129, 1008, 4096), (512, 768, 192),
    (512, 512, 64), (384, 144, 2112), (2048, 4096, 2048),
    (1, 8192, 8192), (4, 8192, 8192), (16, 8192, 8192), (64, 8192, 8192), (3, 1008, 320), (17, 272, 4096), (33, 48, 512),
    (48, 16, 128), (64, 16, 256), (50, 1008, 3072), (5, 8208, 5120), (20, 528, 9216), (64, 4096, 14336),
]


@pytest.mark.parametrize("M,N,K", SHAPES)
def test_preshuffled_gemm_matches_oracle(M, N, K):
    g = torch.Generator().manual_seed(M * 7 + N * 3 + K)
    xq, wq, xs, ws = _problem(M, N, K, g)
    wshuf = mslk_amd.preshuffle_b_mfma(wq.to(DEV))
    y = torch.ops.mslk.f8f8bf16_rowwise_preshuffle(xq.to(DEV), wshuf, xs.to(DEV), ws.to(DEV))
    torch.cuda.synchronize()
    assert y.shape == (M, N) and y.dtype == torch.bfloat16
    assert_gemm_close(y, O.dequant_matmul(xq, wq, xs, ws), f"{M}x{N}x{K}")


@pytest.mark.parametrize("M,N,K", [(512, 512, 256), (300, 272, 384), (16, 512, 512), (40, 304, 1088), (33, 32, 64), (64, 1024, 2048)])
def test_preshuffled_exact_cases_bias_and_fp16(M, N, K):
    g = torch.Generator().manual_seed(K + 5)
    xi = torch.randint(-8, 9, (M, K), generator=g).float()
    wi = torch.randint(-8, 9, (N, K), generator=g).float()
    xs = 2.0 ** torch.randint(-3, 4, (M,), generator=g).float()
    ws = 2.0 ** torch.randint(-3, 4, (N,), generator=g).float()
    bias = torch.randint(-4, 5, (N,), generator=g).float()
    exact = (xi @ wi.T) * xs[:, None] * ws[None, :] + bias[None, :]
    wshuf = mslk_amd.preshuffle_b_mfma(wi.to(F8).to(DEV))
    args = (xi.to(F8).to(DEV), wshuf, xs.to(DEV), ws.to(DEV))
    y = torch.ops.mslk.f8f8bf16_rowwise_preshuffle(*args, bias=bias.to(DEV))
    y16 = torch.ops.mslk.f8f8f16_rowwise_preshuffle(*args, bias=bias.bfloat16().to(DEV))
    torch.cuda.synchronize()
    assert torch.equal(y.cpu(), exact.bfloat16())
    assert y16.dtype == torch.float16 and torch.equal(y16.cpu(), exact.to(torch.float16))


def test_preshuffled_rejects_shapes_the_layout_cannot_hold():
    xq = torch.zeros(8, 64, dtype=F8, device=DEV)
    with pytest.raises(RuntimeError, match="N % 16"):
        torch.ops.mslk.f8f8bf16_rowwise_preshuffle(xq, torch.zeros(24, 64, dtype=F8, device=DEV), torch.ones(8, device=DEV),
                                                   torch.ones(24, device=DEV))
    with pytest.raises(RuntimeError, match="K % 64"):
        torch.ops.mslk.f8f8bf16_rowwise_preshuffle(xq[:, :32].contiguous(), torch.zeros(32, 32, dtype=F8, device=DEV),
                                                   torch.ones(8, device=DEV), torch.ones(32, device=DEV))
