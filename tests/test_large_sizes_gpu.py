"""Operands and outputs beyond 2^31 elements / 4 GiB: every kernel has to form its addresses in 64 bits.
The tensors are made on the GPU; rows on both sides of the 32-bit boundaries (and the first and last
row) are checked against the oracle, bit-exact for the quantizers and to the GEMM tolerance otherwise."""
import pytest
import torch

import mslk_amd
from mslk_amd import moe
from oracle import fp8_rowwise_oracle as O
from tests.helpers import bits32, codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _codes_on_gpu(rows, cols, seed):
    """Random finite e4m3fn codes (|value| < 2^4, both signs) made on the device."""
    g = torch.Generator(device=DEV).manual_seed(seed)
    mag = torch.randint(0, 0x58, (rows, cols), dtype=torch.uint8, device=DEV, generator=g)
    sign = torch.randint(0, 2, (rows, cols), dtype=torch.uint8, device=DEV, generator=g)
    return (mag | (sign << 7)).view(torch.float8_e4m3fn)


def _rows_around(boundary_row, last):
    picks = {0, 1, last - 1, last}
    for r in range(boundary_row - 48, boundary_row + 48):   # enough rows for the normwise error to be a stable statistic
        if 0 <= r <= last:
            picks.add(r)
    return torch.tensor(sorted(picks))


def _check_gemm_rows(y, xq, wq, xs, ws, rows, bias=None):
    ref = O.dequant_matmul(xq[rows.to(DEV)].cpu(), wq.cpu(), xs[rows.to(DEV)].cpu(), ws.cpu(), None if bias is None else bias.cpu())
    max_rel, normwise = O.gemm_errors(y[rows.to(DEV)].float().cpu(), ref)
    assert max_rel <= O.MAX_REL_TOL and normwise <= O.NORMWISE_TOL, (max_rel, normwise)


def test_dense_output_beyond_2_31_elements():
    M, N, K = 66000, 33024, 128                  # M * N = 2.18e9 elements; row 65027 crosses 2^31
    xq, wq = _codes_on_gpu(M, K, 1), _codes_on_gpu(N, K, 2)
    xs = torch.rand(M, device=DEV) + 0.5
    ws = torch.rand(N, device=DEV) + 0.5
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    _check_gemm_rows(y, xq, wq, xs, ws, _rows_around(2**31 // N, M - 1))
    _check_gemm_rows(y, xq, wq, xs, ws, _rows_around(2**32 // (2 * N), M - 1))   # byte offset 2^32
    del y
    torch.cuda.empty_cache()


def test_dense_activations_beyond_4_gib():
    M, N, K = 66000, 256, 65536 + 128            # M * K = 4.33e9 bytes; row 65408 crosses 2^32
    xq, wq = _codes_on_gpu(M, K, 3), _codes_on_gpu(N, K, 4)
    xs = torch.rand(M, device=DEV) * 0.01 + 0.01
    ws = torch.rand(N, device=DEV) + 0.5
    bias = torch.randn(N, device=DEV)
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws, bias)
    torch.cuda.synchronize()
    _check_gemm_rows(y, xq, wq, xs, ws, _rows_around(2**32 // K, M - 1), bias)
    _check_gemm_rows(y, xq, wq, xs, ws, _rows_around(2**31 // K, M - 1), bias)


@pytest.mark.parametrize("M", [3, 40])
def test_skinny_weights_beyond_4_gib(M):
    N, K = 140000, 32768                         # N * K = 4.59e9 bytes; weight row 131072 crosses 2^32
    xq, wq = _codes_on_gpu(M, K, 5), _codes_on_gpu(N, K, 6)
    xs = torch.rand(M, device=DEV) * 0.01 + 0.01
    ws = torch.rand(N, device=DEV) + 0.5
    y = torch.ops.mslk.f8f8bf16_rowwise(xq, wq, xs, ws)
    torch.cuda.synchronize()
    cols = torch.cat([_rows_around(2**32 // K, N - 1), _rows_around(2**31 // K, N - 1)]).unique()
    ref = O.dequant_matmul(xq.cpu(), wq[cols.to(DEV)].cpu(), xs.cpu(), ws[cols.to(DEV)].cpu())
    max_rel, normwise = O.gemm_errors(y[:, cols.to(DEV)].float().cpu(), ref)
    assert max_rel <= O.MAX_REL_TOL and normwise <= O.NORMWISE_TOL, (max_rel, normwise)


def test_grouped_stacked_output_beyond_2_31_elements():
    G, N, K = 4, 33024, 128
    sizes = torch.tensor([20000, 0, 45500, 500], dtype=torch.int64)
    M = int(sizes.sum())
    xq, wq = _codes_on_gpu(M, K, 7), _codes_on_gpu(G * N, K, 8).view(G, N, K)
    xs = torch.rand(M, device=DEV) + 0.5
    ws = torch.rand(G, N, device=DEV) + 0.5
    y = torch.ops.mslk.f8f8bf16_rowwise_grouped_stacked(xq, wq, xs, ws, sizes.to(DEV))
    torch.cuda.synchronize()
    rows = torch.cat([_rows_around(2**31 // N, M - 1), _rows_around(2**32 // (2 * N), M - 1),
                      torch.tensor([19999, 20000, 65499, 65500])]).unique()
    ends = torch.cumsum(sizes, 0)
    for r in rows.tolist():
        g = int(torch.searchsorted(ends, torch.tensor(r), right=True))
        ref = O.dequant_matmul(xq[r:r + 1].cpu(), wq[g].cpu(), xs[r:r + 1].cpu(), ws[g].cpu())
        max_rel, normwise = O.gemm_errors(y[r:r + 1].float().cpu(), ref)
        assert max_rel <= O.MAX_REL_TOL and normwise <= O.NORMWISE_TOL, (r, g, max_rel, normwise)


def test_quantize_beyond_2_32_elements():
    rows, K = 66000, 65536 + 8                   # 4.33e9 elements: codes cross 2^32 bytes at row 65528, input at 32764
    g = torch.Generator(device=DEV).manual_seed(9)
    x = torch.randn(rows, K, device=DEV, dtype=torch.bfloat16, generator=g)
    xq, scale = mslk_amd.quantize_fp8_row(x, use_triton=False)
    torch.cuda.synchronize()
    picks = torch.cat([_rows_around(2**32 // K, rows - 1), _rows_around(2**31 // K, rows - 1),
                       _rows_around(2**30 // K, rows - 1)]).unique()
    rq, rs = O.quantize_fp8_row(x[picks.to(DEV)].cpu())
    assert torch.equal(codes(xq[picks.to(DEV)]), codes(rq))
    assert torch.equal(bits32(scale[picks.to(DEV)]), bits32(rs))
    back = mslk_amd.dequantize_fp8_row(xq, scale)
    torch.cuda.synchronize()
    want = O.dequantize_fp8_row_bf16(rq, rs)
    assert torch.equal(back[picks.to(DEV)].cpu().view(torch.int16), want.view(torch.int16))


def test_fused_producers_beyond_2_31_elements():
    T, D = 140000, 16384                         # T * D = 2.29e9 elements; row 131072 crosses 2^31
    g = torch.Generator(device=DEV).manual_seed(10)
    x = torch.randn(T, 2 * D, device=DEV, dtype=torch.bfloat16, generator=g).clamp_(-2.0, 2.0)
    q, s = moe.silu_mul_quant(x[:, :D], x[:, D:])
    torch.cuda.synchronize()
    picks = torch.cat([_rows_around(2**31 // D, T - 1), _rows_around(2**32 // (4 * D), T - 1)]).unique()
    xc = x[picks.to(DEV)].cpu()
    rq, rs = O.silu_mul_quant(xc[:, :D], xc[:, D:], None)
    assert torch.allclose(s[picks.to(DEV)].cpu(), rs, rtol=2e-6, atol=0)
    got, want = codes(q[picks.to(DEV)]).to(torch.int32), codes(rq).to(torch.int32)
    assert ((got - want).abs() <= 1).all() and (got != want).float().mean().item() <= 2e-4
    del q, s
    # gather: a = T output rows drawn from the same token matrix (first D columns as a contiguous copy)
    xt = x[:, :D].contiguous()
    del x
    torch.cuda.empty_cache()
    token = torch.randperm(T, device=DEV, generator=g).to(torch.int32)
    expert = torch.randint(0, 2, (T,), device=DEV, generator=g)
    scores = torch.rand(T, 2, device=DEV, generator=g) + 0.5
    q, s = moe.gather_scale_quant_dense_tokens(xt, token, expert, scores)
    torch.cuda.synchronize()
    # output rows around the boundary, and output rows whose SOURCE row lies around it
    src_hit = torch.nonzero((token.cpu().long() - 2**31 // D).abs() <= 2).flatten()
    picks = torch.cat([picks, src_hit]).unique()
    tok_c, exp_c = token.cpu()[picks].long(), expert.cpu()[picks]
    rq, rs = O.gather_scale_quant_dense_tokens(xt[tok_c.to(DEV)].cpu(), torch.arange(len(picks)), exp_c,
                                               scores.cpu()[tok_c], None)
    assert torch.equal(codes(q[picks.to(DEV)]), codes(rq))
    assert torch.equal(bits32(s[picks.to(DEV)]), bits32(rs))
