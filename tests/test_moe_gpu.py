"""GPU parity of the fused producers of quantized MoE activations.  Shapes and options follow
test/moe/activation_test.py:97-170 and test/moe/gather_scatter_test.py:128-215.

gather_scale_quant_dense_tokens has no transcendental: codes and scales must equal the oracle's bit
for bit.  silu_mul_quant evaluates a sigmoid whose last bits differ between implementations, so a
value next to a rounding boundary may land on the neighbouring code: the dequantized result is held
to the reference test's tolerance and the differing codes are bounded in number and distance."""
import pytest
import torch

import mslk_amd
from mslk_amd import moe
from oracle import fp8_rowwise_oracle as O
from tests.helpers import bits32, codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
SENT = 0x55


def _code_distance(a, b):
    """Distance in representable values between two e4m3fn code tensors (sign-magnitude -> ordinal)."""
    def ordinal(c):
        c = c.to(torch.int32)
        mag = c & 0x7F
        return torch.where((c & 0x80) != 0, -mag, mag)
    return (ordinal(a) - ordinal(b)).abs()


@pytest.mark.parametrize("T,D,ub,contiguous,partial,dtype", [
    (1, 5120, None, True, False, torch.bfloat16), (128, 5120, 1200.0, False, True, torch.bfloat16),
    (2048, 7168, None, False, False, torch.bfloat16), (4096, 5120, 0.05, True, True, torch.bfloat16),
    (300, 2048, None, True, False, torch.float16), (64, 16384, None, True, False, torch.bfloat16),
    (9, 20000, 1200.0, True, False, torch.bfloat16), (33, 1001, None, True, True, torch.bfloat16),
    (16384, 5120, None, False, False, torch.bfloat16),
    # rows of MoE intermediate sizes in large numbers: one wavefront per row
    (4099, 768, None, True, True, torch.bfloat16), (2048, 1408, 1200.0, False, False, torch.bfloat16),
    (3001, 2048, None, True, False, torch.float16), (5000, 128, None, False, True, torch.bfloat16),
    (2050, 520, 0.05, True, False, torch.bfloat16), (2047, 768, None, True, False, torch.bfloat16),
])
def test_silu_mul_quant(T, D, ub, contiguous, partial, dtype):
    g = torch.Generator().manual_seed(T + D)
    x = torch.randn(T, 2 * D, generator=g)
    x = (torch.sign(x) * torch.clamp(x.abs(), 0.01, 2.0)).to(dtype)     # the reference test's input distribution
    xd = x.to(DEV)
    x0, x1 = xd[:, :D], xd[:, D:]
    if contiguous:
        x0, x1 = x0.contiguous(), x1.contiguous()
    n_valid = T // 2 if partial else T
    cnt = torch.tensor([n_valid], dtype=torch.int32, device=DEV) if partial else None
    ubt = None if ub is None else torch.tensor([ub], dtype=torch.float32)
    # pre-fill the outputs through the allocator so untouched rows are recognisable
    q, s = moe.silu_mul_quant(x0, x1, None if ubt is None else ubt.to(DEV), cnt)
    torch.cuda.synchronize()
    assert q.shape == (T, D) and q.dtype == torch.float8_e4m3fn and s.shape == (T,)
    rq, rs = O.silu_mul_quant(x[:n_valid, :D], x[:n_valid, D:], ubt)
    got_q, got_s = codes(q)[:n_valid], s.cpu()[:n_valid]
    # scales: the row maximum goes through one sigmoid, so allow a few fp32 ulps
    assert torch.allclose(got_s, rs, rtol=2e-6, atol=0)
    dist = _code_distance(got_q, codes(rq))
    assert dist.max().item() <= 1
    assert (dist != 0).float().mean().item() <= 2e-4
    # the reference test's own criterion
    y, y_ref = got_q.view(torch.float8_e4m3fn).float() * got_s[:, None], rq.float() * rs[:, None]
    torch.testing.assert_close(y, y_ref, rtol=1e-1, atol=1e-3)


def test_silu_mul_quant_skips_invalid_rows_and_matches_two_step_path():
    g = torch.Generator().manual_seed(3)
    T, D = 256, 5120
    x0 = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    x1 = torch.randn(T, D, generator=g).bfloat16().to(DEV)
    L = mslk_amd._lib.lib()
    out = torch.full((T, D), SENT, dtype=torch.uint8, device=DEV)
    sc = torch.full((T,), -1.0, device=DEV)
    cnt = torch.tensor([100], dtype=torch.int64, device=DEV)
    mslk_amd._lib.check(L.mslk_amd_silu_mul_quant(x0.data_ptr(), x1.data_ptr(), 0, T, D, D, D, out.data_ptr(), sc.data_ptr(),
                                                  None, cnt.data_ptr(), 0, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert (out[100:] == SENT).all() and (sc[100:] == -1.0).all()
    assert (sc[:100] > 0).all()
    # the fused kernel against fp32 silu*mul computed by torch on the GPU followed by a saturating quantization
    y = (x0.float() * torch.sigmoid(x0.float()) * x1.float()).cpu()
    rq, rs = O.quantize_rows_saturating(y[:100])
    dist = _code_distance(out[:100].cpu(), codes(rq))
    assert dist.max().item() <= 1 and (dist != 0).float().mean().item() <= 2e-4


@pytest.mark.parametrize("E,T,D,partial,rowmajor,xdtype,sdtype,idx", [
    (2, 1, 5120, False, True, torch.bfloat16, torch.bfloat16, torch.int32),
    (8, 128, 5120, True, False, torch.bfloat16, torch.bfloat16, torch.int32),
    (8, 4096, 5120, False, False, torch.bfloat16, torch.bfloat16, torch.int64),
    (2, 4096, 5120, True, True, torch.bfloat16, torch.float32, torch.int32),
    (4, 300, 7168, False, True, torch.float16, torch.float16, torch.int64),
    (3, 40, 1001, False, True, torch.bfloat16, torch.float32, torch.int32),
    (2, 16, 20000, False, False, torch.bfloat16, torch.bfloat16, torch.int32),
    (8, 4099, 768, True, False, torch.bfloat16, torch.bfloat16, torch.int32),
    (4, 2048, 1408, False, True, torch.bfloat16, torch.float32, torch.int64),
    (2, 3001, 2048, True, True, torch.float16, torch.float16, torch.int32),
    (3, 6000, 136, False, False, torch.bfloat16, torch.bfloat16, torch.int32),
])
def test_gather_scale_quant_bit_exact(E, T, D, partial, rowmajor, xdtype, sdtype, idx):
    g = torch.Generator().manual_seed(E * 1000 + T + D)
    x = torch.randn(T, D, generator=g).to(xdtype)
    expert = torch.randint(0, E, (T,), generator=g)                  # int64, as torch.randint gives
    token = torch.randperm(T, generator=g).to(idx)
    scores_et = torch.randn(E, T, generator=g).to(sdtype)              # the reference keeps scores as [E, T]
    ub = torch.tensor([1200.0])
    n_valid = T // 2 if partial else T
    cnt = torch.tensor([n_valid], dtype=torch.int32, device=DEV) if partial else None
    tok_in, exp_in = token.clone(), expert.clone()
    if partial:   # as the reference test: indices beyond the valid count are -1
        tok_in[n_valid:] = -1
        exp_in[n_valid:] = -1
    scores_dev = scores_et.to(DEV).contiguous().transpose(0, 1)       # [T, E] view with strides (1, T)
    if rowmajor:
        scores_dev = scores_dev.contiguous()
    q, s = moe.gather_scale_quant_dense_tokens(x.to(DEV), tok_in.to(DEV), exp_in.to(DEV), scores_dev, ub.to(DEV), cnt)
    torch.cuda.synchronize()
    assert q.shape == (T, D) and s.shape == (T,)
    rq, rs = O.gather_scale_quant_dense_tokens(x, token[:n_valid], expert[:n_valid], scores_et.t(), ub)
    assert torch.equal(codes(q)[:n_valid], codes(rq))
    assert torch.equal(bits32(s)[:n_valid], bits32(rs))


def test_gather_out_of_range_indices_touch_nothing():
    T, D, E = 8, 256, 2
    x = torch.randn(T, D).bfloat16().to(DEV)
    tok = torch.tensor([0, 9, -1, 3], dtype=torch.int32, device=DEV)
    exp = torch.tensor([0, 0, 0, 5], dtype=torch.int64, device=DEV)
    scores = torch.ones(T, E, device=DEV)
    L = mslk_amd._lib.lib()
    out = torch.full((4, D), SENT, dtype=torch.uint8, device=DEV)
    sc = torch.full((4,), -1.0, device=DEV)
    mslk_amd._lib.check(L.mslk_amd_gather_scale_quant_dense_tokens(
        x.data_ptr(), 0, T, D, tok.data_ptr(), 1, exp.data_ptr(), 0, 4, scores.data_ptr(), 2, E, E, 1, out.data_ptr(),
        sc.data_ptr(), None, None, 0, torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    assert (out[1:] == SENT).all() and (sc[1:] == -1.0).all() and sc[0] > 0


def test_fused_producers_feed_the_gemm():
    """gather -> GEMM -> silu_mul_quant -> GEMM: the chain the MoE layer runs (mslk/moe/layers.py:811-965),
    checked end to end against the oracle chain on the oracle's own quantized activations."""
    g = torch.Generator().manual_seed(11)
    T, D, H, E = 96, 512, 1024, 2
    x = torch.randn(T, D, generator=g).bfloat16()
    scores = torch.rand(T, E, generator=g) + 0.5
    token, expert = torch.randperm(T, generator=g).to(torch.int32), torch.zeros(T, dtype=torch.int64)
    w13 = (torch.randn(2 * H, D, generator=g) * 0.05).bfloat16()
    w2 = (torch.randn(D, H, generator=g) * 0.05).bfloat16()
    w13q, w13s = O.quantize_fp8_row(w13)
    w2q, w2s = O.quantize_fp8_row(w2)
    xq, xs = moe.gather_scale_quant_dense_tokens(x.to(DEV), token.to(DEV), expert.to(DEV), scores.to(DEV))
    h = torch.ops.mslk.f8f8bf16_rowwise(xq, w13q.to(DEV), xs, w13s.to(DEV))
    hq, hs = moe.silu_mul_quant(h[:, :H], h[:, H:])
    y = torch.ops.mslk.f8f8bf16_rowwise(hq, w2q.to(DEV), hs, w2s.to(DEV))
    torch.cuda.synchronize()
    rxq, rxs = O.gather_scale_quant_dense_tokens(x, token, expert, scores)
    assert torch.equal(codes(xq), codes(rxq))
    ref = O.dequant_matmul(hq.cpu(), w2q, hs.cpu(), w2s)
    max_rel, normwise = O.gemm_errors(y.float().cpu(), ref)
    assert max_rel <= O.MAX_REL_TOL and normwise <= O.NORMWISE_TOL
