"""GPU parity of the HIP row quantizer against the oracle: codes and scales bit for bit.
Shapes follow the reference's tests (test/quantize/triton/fp8_quantize_test.py:139-220,
test/quantize/fp8_quantize_correctness_test.py:60-124)."""
import pytest
import torch

import mslk_amd
from mslk_amd import _lib
from oracle import c_twin
from oracle import fp8_rowwise_oracle as O
from tests.helpers import assert_quant_bit_exact, bits32, codes

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
ALL_BF16 = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def _run(a_cpu, scale_ub=None, align=None):
    ub = None if scale_ub is None else scale_ub.to(DEV)
    xq, s = mslk_amd.quantize_fp8_row(a_cpu.to(DEV), scale_ub=ub, align_rows_to=align, use_triton=False)
    torch.cuda.synchronize()
    return xq, s


def test_hw_cast_sweep_matches_oracle():
    """Device conversion routine vs the C twin: every fp32 with a zero low mantissa half (all
    exponents, signs, 7 mantissa bits x 512 patterns) plus dense random bits and the 448..480 edge."""
    g = torch.Generator().manual_seed(1)
    hi = torch.arange(65536, dtype=torch.int64)
    lo_patterns = torch.tensor([0x0000, 0x0001, 0x7FFF, 0x8000, 0x8001, 0xFFFF, 0x4000, 0xC000], dtype=torch.int64)
    bits = ((hi[:, None] << 16) | lo_patterns[None, :]).reshape(-1)
    rnd = torch.randint(0, 2**32, (8_000_000,), generator=g, dtype=torch.int64)
    edge = torch.linspace(440.0, 482.0, 200001).view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    allbits = torch.cat([bits, rnd, edge, edge | 0x80000000])
    x = (allbits & 0xFFFFFFFF).to(torch.int64)
    x = torch.where(x >= 2**31, x - 2**32, x).to(torch.int32).view(torch.float32)
    out = torch.empty(x.numel(), dtype=torch.uint8, device=DEV)
    xd = x.to(DEV)
    _lib.check(_lib.lib().mslk_amd_debug_cast_e4m3fn(xd.data_ptr(), x.numel(), out.data_ptr(), None))
    torch.cuda.synchronize()
    want = c_twin.e4m3fn_cast(x)
    got = out.cpu()
    nan = torch.isnan(x)
    assert torch.equal(got[~nan], want[~nan])
    assert ((got[nan] & 0x7F) == 0x7F).all()


def test_every_bf16_amax_and_every_bf16_value():
    # scales: every positive finite bf16 as a one-element row (tests the device 1/x and the eps clamp)
    a = ALL_BF16[1:0x7F80].reshape(-1, 1).contiguous()
    xq, s = _run(a)
    assert_quant_bit_exact(a, xq, s)
    # codes: rows holding every finite bf16 up to amax, for a spread of amax values
    fin = ALL_BF16[torch.isfinite(ALL_BF16.float())]
    rows = []
    for b in list(range(0x3F00, 0x4000, 3)) + [0x0001, 0x0080, 0x2B8D, 0x2B8E, 0x3380, 0x4700, 0x7F7F]:
        amax = torch.tensor([b], dtype=torch.int16).view(torch.bfloat16).float().item()
        rows.append(fin[fin.float().abs() <= amax])
    K = (max(r.numel() for r in rows) + 7) // 8 * 8
    a = torch.zeros(len(rows), K, dtype=torch.bfloat16)
    for i, r in enumerate(rows):
        a[i, : r.numel()] = r
    xq, s = _run(a)
    assert_quant_bit_exact(a, xq, s)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_reference_shape_sweep(dtype):
    g = torch.Generator().manual_seed(2)
    shapes = [(2, n) for n in range(1, 9000, 100)]
    shapes += [(16, 16), (64, 512), (1024, 1024), (4096, 2048), (8192, 4096), (333, 777), (1, 128), (128, 1),
               (5, 8192), (3, 16384), (2, 40000), (2, 70008), (2500, 8192), (64, 8192), (1, 8192), (5, 65536), (3, 57344),
               (2, 32776), (2, 65544)]
    for shape in shapes:
        a = torch.randn(shape, generator=g).to(dtype)
        xq, s = _run(a)
        assert_quant_bit_exact(a, xq, s)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_many_short_rows(dtype):
    """4096 rows and more of K <= 256 (per-head quantization): 8 / 16 / 32 lanes per row, several rows per wavefront.
    Ragged row counts, K on both sides of each team width, scale_ub, padded output rows, a jagged batch."""
    g = torch.Generator().manual_seed(12)
    for rows, K in [(4096, 8), (4099, 64), (5000, 72), (4097, 128), (6001, 136), (4100, 256), (4096, 16), (8200, 120),
                    (4101, 200), (4096, 264)]:
        a = (torch.randn(rows, K, generator=g) * torch.logspace(-3, 3, rows)[:, None]).to(dtype)
        a[7] = 0
        xq, s = _run(a)
        assert_quant_bit_exact(a, xq, s)
    a = (torch.randn(4500, 128, generator=g) * 3).to(dtype)
    t = torch.tensor([1.5], dtype=torch.float32)
    xq, s = _run(a, scale_ub=t)
    assert_quant_bit_exact(a, xq, s, scale_ub=t)
    a = torch.randn(4200, 100 if dtype != torch.float32 else 104, generator=g).to(dtype)
    if a.shape[1] % 8 == 0:
        xq, s = _run(a, align=16)
        assert_quant_bit_exact(a, xq, s, K_out=112)
    b = torch.randn(8, 600, 128, generator=g).to(dtype)          # 4800 rows in 8 groups, some rows dead
    zs = torch.tensor([600, 0, 1, 599, 300, 17, 600, 64], dtype=torch.int64)
    xq, s = mslk_amd.quantize_fp8_row(b.to(DEV), zero_start_index_M=zs.to(DEV), use_triton=False)
    torch.cuda.synchronize()
    rq, rs = O.quantize_fp8_row_jagged(b, zs)
    assert torch.equal(codes(xq), codes(rq)) and torch.equal(bits32(s), bits32(rs))


def test_special_rows_and_magnitudes():
    g = torch.Generator().manual_seed(3)
    a = (torch.randn(512, 2048, generator=g) * torch.logspace(-20, 20, 512)[:, None]).to(torch.bfloat16)
    a[0] = 0
    a[1, 5] = float("nan")
    a[2] = -0.0
    a[3, 100] = float("inf")
    a[4] = 1e-39          # bf16 subnormals
    a[5] = 3.3895313892515355e38
    a[6, :] = 0; a[6, 77] = -5.0
    xq, s = _run(a)
    assert_quant_bit_exact(a, xq, s)
    assert codes(xq)[2].eq(0x80).all()
    assert s[0].item() == 2.236306529429413e-15
    for dtype, zero_scale in ((torch.float16, 1.0), (torch.float32, 2.2321429389771845e-15)):
        z = torch.zeros(4, 256, dtype=dtype)
        xq, s = _run(z)
        assert_quant_bit_exact(z, xq, s)
        assert s[0].item() == zero_scale


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_scale_ub(dtype):
    g = torch.Generator().manual_seed(4)
    for shape in [(64, 1024), (7, 777), (2500, 4096)]:
        a = (torch.randn(shape, generator=g) * 3).to(dtype)
        for ub in (1200.0, 1.2345, 0.0):
            t = torch.tensor([ub], dtype=torch.float32)
            xq, s = _run(a, scale_ub=t)
            assert_quant_bit_exact(a, xq, s, scale_ub=t)


def test_batched_strided_and_padded_inputs():
    g = torch.Generator().manual_seed(5)
    for shape in [(3, 64, 512), (2, 3, 17, 136), (4, 1, 8)]:
        a = torch.randn(shape, generator=g).bfloat16()
        xq, s = _run(a)
        assert xq.shape == a.shape and s.shape == a.shape[:-1]
        assert_quant_bit_exact(a, xq, s)
    base = torch.randn(300, 1000, generator=g).bfloat16()
    for view in (base[:, :512], base[:, 8:520], base[::2, 3:77], base.t(), base[:, 1:]):
        xq, s = _run(view)
        assert_quant_bit_exact(view.contiguous(), xq, s)
    for K, align in [(100, 16), (777, 8), (4096, 16), (130, 128)]:
        a = torch.randn(33, K, generator=g).bfloat16()
        xq, s = _run(a, align=align)
        K_out = (K + align - 1) // align * align
        assert_quant_bit_exact(a, xq, s, K_out=K_out)


def test_legacy_name_and_errors():
    a = torch.randn(8, 64).bfloat16()
    xq, s = mslk_amd.quantize_fp8_per_row(a.to(DEV))
    assert_quant_bit_exact(a, xq, s)
    with pytest.raises(RuntimeError, match="one entry per group"):
        mslk_amd.quantize_fp8_row(a.to(DEV), zero_start_index_M=torch.zeros(8, dtype=torch.int64, device=DEV))
    with pytest.raises(RuntimeError, match="int64 or int32"):
        mslk_amd.quantize_fp8_row(a.to(DEV), zero_start_index_M=torch.zeros(1, device=DEV))
    with pytest.raises(RuntimeError):
        mslk_amd.quantize_fp8_row(torch.zeros(4, 0, dtype=torch.bfloat16, device=DEV))
    xq, s = mslk_amd.quantize_fp8_row(torch.zeros(0, 64, dtype=torch.bfloat16, device=DEV))
    assert xq.shape == (0, 64) and s.shape == (0,)


def test_round_trip_and_full_size_properties():
    """cfg2-sized activations (8192 x 4096 with outlier channels): bit-exact against the oracle and the
    size-independent properties (every row holds +-448, dequantization error within half an ulp)."""
    from mslk_amd import workloads as W
    wl = W.cfg1(M=8192)
    xq, s = _run(wl.x)
    assert_quant_bit_exact(wl.x, xq, s)
    c = codes(xq)
    assert ((c & 0x7F) == 0x7E).any(dim=1).all()
    deq = xq.float().cpu() * s.cpu()[:, None]
    assert torch.allclose(deq, wl.x.float(), atol=2e-1, rtol=1e-1)  # the reference's own round-trip bound


@pytest.mark.parametrize("shape,align,idx_dtype", [
    ((20, 30), None, torch.int64), ((20, 30), 16, torch.int64), ((6, 4, 2, 3), None, torch.int64),
    ((4, 2, 3), None, torch.int32), ((8, 40, 512), None, torch.int64), ((3, 2, 300, 1024), None, torch.int32),
    ((2, 2500, 4096), None, torch.int64), ((5, 9, 20000), None, torch.int64), ((16, 64, 136), 128, torch.int64),
])
def test_jagged_rows(shape, align, idx_dtype):
    """Shapes of test/quantize/triton/fp8_quantize_test.py:201-222 plus every kernel variant."""
    g = torch.Generator().manual_seed(sum(shape))
    a = torch.randn(shape, generator=g).bfloat16()
    groups = 1
    for d in shape[:-2]:
        groups *= d
    zs = torch.randint(0, shape[-2] + 1, (groups,), generator=g).to(idx_dtype)
    zs[0] = shape[-2]      # one full group
    if groups > 1:
        zs[-1] = 0         # one empty group
    # poison the rows that must not be read: a NaN there would change the result if it were
    poisoned = a.clone().view(groups, shape[-2], shape[-1])
    for gi in range(groups):
        poisoned[gi, int(zs[gi]):] = float("nan")
    xq, s = mslk_amd.quantize_fp8_row(poisoned.view(shape).to(DEV), zero_start_index_M=zs.to(DEV), align_rows_to=align,
                                       use_triton=False)
    torch.cuda.synchronize()
    rq, rs = O.quantize_fp8_row_jagged(a, zs)
    K = shape[-1]
    got = codes(xq)
    if align is not None:
        K_out = (K + align - 1) // align * align
        assert got.shape[-1] == K_out and (got[..., K:] == 0).all()
        got = got[..., :K]
    assert torch.equal(got, codes(rq))
    assert torch.equal(bits32(s), bits32(rs))
    assert s.shape == a.shape[:-1]


@pytest.mark.parametrize("shape", [(1, 256), (3, 16), (7, 777), (64, 1024), (2, 3, 17, 136), (2500, 4096), (5, 3), (300, 4104),
                                   (4096, 520), (33, 8), (1000, 1000), (300, 4100), (33, 7), (2, 9), (513, 1001)])
def test_dequantize_bit_exact(shape):
    g = torch.Generator().manual_seed(sum(shape))
    rows = 1
    for d in shape[:-1]:
        rows *= d
    q = torch.randint(0, 256, shape, generator=g, dtype=torch.uint8)
    if shape == (1, 256):
        q = torch.arange(256, dtype=torch.uint8).reshape(1, 256)    # every code, NaNs included
    q = q.view(torch.float8_e4m3fn)
    sc = torch.rand(shape[:-1], generator=g) * 4 + 2.0 ** -12
    out = mslk_amd.dequantize_fp8_row(q.to(DEV), sc.to(DEV))
    torch.cuda.synchronize()
    ref = O.dequantize_fp8_row_bf16(q, sc)
    assert out.shape == q.shape and out.dtype == torch.bfloat16
    o16, r16 = out.cpu().view(torch.int16), ref.view(torch.int16)
    nan = torch.isnan(ref.float())
    assert torch.isnan(out.cpu().float()[nan]).all()
    assert torch.equal(o16[~nan], r16[~nan])


def test_dequantize_round_trip_full_size():
    g = torch.Generator().manual_seed(12)
    a = torch.randn(4096, 4096, generator=g).bfloat16().to(DEV)
    xq, s = mslk_amd.quantize_fp8_row(a, use_triton=False)
    back = mslk_amd.dequantize_fp8_row(xq, s).float()
    af = a.float()
    assert ((back - af).abs() <= af.abs() * 2.0 ** -4 + af.abs().amax(dim=1, keepdim=True) * 2.0 ** -9).all()
    # dequantize(quantize(.)) is idempotent: quantizing the result again reproduces codes and values
    xq2, s2 = mslk_amd.quantize_fp8_row(back.bfloat16(), use_triton=False)
    back2 = mslk_amd.dequantize_fp8_row(xq2, s2).float()
    assert (back2 - back).abs().max() <= back.abs().max() * 2.0 ** -7


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16, torch.float32])
def test_triton_arithmetic_mode(dtype):
    """`use_triton=True` (the default, as in the reference): codes and scales equal the oracle's restatement of the
    reference's Triton kernel bit for bit (IEEE divisions on both sides), over the reference's shape sweep, eps variants,
    scale_ub, jagged rows and padding; `use_triton=False` gives the torch emulation."""
    g = torch.Generator().manual_seed(17)
    for shape in [(1, 16), (7, 777), (64, 1024), (2500, 4096), (3, 5, 136), (5, 20000)]:
        a = (torch.randn(shape, generator=g) * 3).to(dtype)
        a.view(-1, shape[-1])[0].zero_()                        # a zero row: the eps clamp decides
        a.view(-1, shape[-1])[-1].mul_(2.0 ** -14)               # a row below 1/512
        for eps_opt, ub in [(1.0 / 512.0, None), (None, None), (1e-4, 1.2345), (1.0 / 512.0, 1200.0)]:
            ubt = None if ub is None else torch.tensor([ub], dtype=torch.float32)
            xq, s = mslk_amd.quantize_fp8_row(a.to(DEV), scale_ub=None if ubt is None else ubt.to(DEV), eps_opt=eps_opt)
            torch.cuda.synchronize()
            rq, rs = O.quantize_fp8_row_triton_arithmetic(a, ubt, eps_opt if eps_opt is not None else 1e-12)
            assert torch.equal(codes(xq), codes(rq)), (shape, eps_opt, ub)
            assert torch.equal(bits32(s), bits32(rs)), (shape, eps_opt, ub)
    # use_triton=False selects the torch branch, and so does the legacy operator
    a = torch.randn(33, 256, generator=g).to(dtype)
    xq, s = mslk_amd.quantize_fp8_row(a.to(DEV), use_triton=False)
    assert_quant_bit_exact(a, xq, s)
    xq, s = torch.ops.mslk.quantize_fp8_per_row(a.to(DEV))
    assert_quant_bit_exact(a, xq, s)
    # jagged + padding
    a = torch.randn(4, 6, 40, generator=g).to(dtype)
    zs = torch.tensor([6, 0, 3, 1])
    xq, s = mslk_amd.quantize_fp8_row(a.to(DEV), zero_start_index_M=zs.to(DEV), align_rows_to=16)
    masked = a.clone()
    for gi in range(4):
        masked[gi, int(zs[gi]):] = 0
    rq, rs = O.quantize_fp8_row_triton_arithmetic(masked)
    assert torch.equal(codes(xq)[..., :40], codes(rq)) and (codes(xq)[..., 40:] == 0).all()
    assert torch.equal(bits32(s), bits32(rs))


def test_default_arithmetic_saturates_under_scale_ub():
    """A GPU caller of the reference gets its Triton kernel by default, which stores +-448 where `scale_ub` cuts the row
    maximum (fp8_quantize.py:142-144,164-166); the torch emulation stores NaN codes there."""
    a = torch.tensor([[1.0, -2.0, 1000.0, -3000.0] * 16], dtype=torch.bfloat16)
    ub = torch.tensor([2.0], device=DEV)
    xq, s = mslk_amd.quantize_fp8_row(a.to(DEV), scale_ub=ub)
    c = codes(xq)[0, :4].tolist()
    assert c == [0x76, 0xFE, 0x7E, 0xFE], [hex(v) for v in c]     # 1 / (2 / 448) = 224, -448, +448 (saturated), -448
    assert s.cpu().item() == (torch.tensor(2.0) / 448.0).item()    # fl32(2 / 448)
    xq, s = mslk_amd.quantize_fp8_row(a.to(DEV), scale_ub=ub, use_triton=False)
    assert (codes(xq)[0, 2:4] & 0x7F).tolist() == [0x7F, 0x7F]   # no saturation in the torch emulation
